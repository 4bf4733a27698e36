// Layer-list models on the host side: config.json + model.safetensors -> ps_hip_seq (include/ps_hip.h, "layer-list models"), with the same
// generation entry points as Model (greedy on the device, or every step's logits through a SamplerChain).  The architecture named in
// config.json selects the function that maps configuration and tensors onto layer descriptors (seq_architectures()).
#pragma once
#include "json_gguf.hpp"
#include "sampler.hpp"
#include "../../../include/ps_hip.h"

#include <deque>
#include <functional>
#include <map>
#include <span>

namespace powerserve {

struct SafeTensor {
    std::string dtype; // "BF16", "F32", "I32"
    std::vector<int64_t> shape;
    const void *data = nullptr;
    size_t nbytes = 0;
    int64_t numel() const { int64_t n = 1; for (auto s : shape) n *= s; return n; }
};
// an 8-byte little-endian header length, the JSON header (name -> dtype, shape, data_offsets), the data; memory-mapped, nothing is executed
struct SafeTensorsFile {
    explicit SafeTensorsFile(const std::string &path);
    ~SafeTensorsFile();
    SafeTensorsFile(const SafeTensorsFile &) = delete;
    const SafeTensor &at(const std::string &name) const;
    bool contains(const std::string &name) const { return tensors.count(name) != 0; }
    std::vector<float> f32(const std::string &name) const;            // any float tensor widened to fp32
    std::vector<uint16_t> bf16_bits(const std::string &name) const;   // a bfloat16 matrix's bit patterns
    std::map<std::string, SafeTensor> tensors;

private:
    std::string m_path;
    void *m_map = nullptr;
    size_t m_size = 0;
};

// puts tensors on the device and keeps them until the model goes
struct SeqUploader {
    ps_hip_ctx *ctx;
    bool as_f32;
    std::vector<void *> vecs;
    std::vector<ps_dense *> mats;
    std::deque<ps_seq_layer> beside; // descriptors of second mixers, pointed to from the layers (addresses stay put)
    const float *vec(const std::vector<float> &a);
    const ps_dense *mat(const std::vector<uint16_t> &bits, int64_t rows, int64_t cols);
    void free_all();
};

struct SeqModel {
    SeqModel(const std::string &model_dir, const std::string &dtype, int device, size_t max_batch, int n_slots, int max_context = 0);
    ~SeqModel();
    SeqModel(const SeqModel &) = delete;
    int acquire();
    void release(int slot);
    int64_t position(int slot) const;
    // the next tokens of the sequence in `slot`; logits of the wanted places, [want.size()][vocab]
    std::vector<float> forward(int slot, const std::vector<Token> &tokens, const std::vector<int> &want);
    // prefill all but the last prompt token, then `steps` tokens: arg-max on the device / each step's logits through the chain
    std::vector<Token> generate(const std::vector<Token> &prompt, int steps);
    std::vector<Token> generate(const std::vector<Token> &prompt, int steps, SamplerChain &sampler);
    std::string arch;
    uint32_t vocab = 0, width = 0, n_layers = 0;

private:
    ps_hip_ctx *m_ctx = nullptr;
    ps_hip_seq *m_h = nullptr;
    SeqUploader m_up{};
};

using SeqArchitecture = std::function<void(const JsonValue &cfg, const SafeTensorsFile &st, SeqUploader &up, std::vector<ps_seq_layer> &layers, ps_seq_desc &d)>;
const std::map<std::string, SeqArchitecture> &seq_architectures();
bool is_seq_model_dir(const std::string &model_dir);
auto load_seq_model(const std::string &model_dir, const std::string &dtype = "bfloat16", int device = 0, size_t max_batch = 256, int n_slots = 2,
                    int max_context = 0) -> std::shared_ptr<SeqModel>;

} // namespace powerserve
