// Whisper audio encoder on the gfx950 backend: the encoder half of the reference's
// examples/whisper_poc.cpp (:57-141), same module tree and HuggingFace parameter names
// ("model.encoder.*"), loaded from a .safetensors file and run as lazy GPU graphs.
//
//   whisper_encoder <model.safetensors> [--layers N] [--heads H] [--dtype f32|f16|bf16]
//                   [--mel <file.safetensors>] [--out <file.bin>] [--repeat R]
//
// --mel names a safetensors file holding "mel" (batch, n_mels, n_frames); without it a seeded
// random spectrogram of 3000 frames is used.  --out receives the encoder output as raw
// little-endian float32 (batch, n_frames / 2, d_model).  d_model, n_mels, ffn width and the
// number of positions are read off the weights.
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <string>

#include "axiom/axiom.hpp"

using namespace axiom;
using namespace axiom::nn;

struct WhisperEncoderLayer : Module {
    MultiHeadAttention self_attn_;
    LayerNorm self_attn_layer_norm_;
    Linear fc1_{true}, fc2_{true};
    LayerNorm final_layer_norm_;

    explicit WhisperEncoderLayer(int num_heads) : self_attn_(num_heads) {
        register_module("self_attn", self_attn_);
        register_module("self_attn_layer_norm", self_attn_layer_norm_);
        register_module("fc1", fc1_);
        register_module("fc2", fc2_);
        register_module("final_layer_norm", final_layer_norm_);
    }
    Tensor forward(const Tensor &x) const override { // pre-norm attention and MLP, each with a residual
        Tensor h = self_attn_layer_norm_(x);
        h = ops::add(x, self_attn_.forward(h, h, h));
        Tensor m = fc2_(fc1_(final_layer_norm_(h)).gelu());
        return ops::add(h, m);
    }
};

struct WhisperEncoder : Module {
    Conv1d conv1_{1, 1}, conv2_{2, 1};
    Embedding embed_positions_;
    ModuleList layers_;
    LayerNorm layer_norm_;

    WhisperEncoder(int n_layers, int n_heads) {
        register_module("conv1", conv1_);
        register_module("conv2", conv2_);
        register_module("embed_positions", embed_positions_);
        register_module("layers", layers_);
        register_module("layer_norm", layer_norm_);
        for (int i = 0; i < n_layers; ++i) layers_.emplace_back<WhisperEncoderLayer>(n_heads);
    }
    Tensor forward(const Tensor &mel) const override { // (batch, n_mels, n_frames)
        Tensor x = conv2_(conv1_(mel).gelu()).gelu().transpose({0, 2, 1}); // (batch, n_frames / 2, d_model)
        const Tensor positions = Tensor::arange(0, static_cast<int64_t>(x.shape()[1])).gpu();
        x = ops::add(x, embed_positions_(positions));
        for (size_t i = 0; i < layers_.size(); ++i) x = layers_[i].forward(x);
        return layer_norm_(x);
    }
};

int main(int argc, char **argv) {
    if (argc < 2) {
        fprintf(stderr, "usage: %s <model.safetensors> [--layers N] [--heads H] [--dtype f32|f16|bf16] [--mel file] [--out file] [--repeat R]\n", argv[0]);
        return 2;
    }
    int layers = 4, heads = 6, repeat = 1;
    std::string dtype = "f32", mel_path, out_path;
    for (int i = 2; i + 1 < argc; i += 2) {
        const std::string k = argv[i], v = argv[i + 1];
        if (k == "--layers") layers = std::atoi(v.c_str());
        else if (k == "--heads") heads = std::atoi(v.c_str());
        else if (k == "--dtype") dtype = v;
        else if (k == "--mel") mel_path = v;
        else if (k == "--out") out_path = v;
        else if (k == "--repeat") repeat = std::atoi(v.c_str());
        else { fprintf(stderr, "unknown option %s\n", k.c_str()); return 2; }
    }
    const DType dt = dtype == "bf16" ? DType::BFloat16 : dtype == "f16" ? DType::Float16 : DType::Float32;
    try {
        if (!system::is_gpu_available()) throw DeviceError("no gfx950 device");
        auto t0 = std::chrono::steady_clock::now();
        auto state = io::safetensors::load(argv[1], Device::GPU);
        WhisperEncoder enc(layers, heads);
        enc.load_state_dict(state, "model.encoder.", /*strict=*/false); // k_proj has no bias in Whisper
        enc.to(dt);
        const size_t n_mels = state.at("model.encoder.conv1.weight").shape()[1], d_model = state.at("model.encoder.conv1.weight").shape()[0];
        const double load_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();

        Tensor mel;
        if (!mel_path.empty()) mel = io::safetensors::load_tensor(mel_path, "mel", Device::GPU);
        else {
            Tensor::manual_seed(42);
            mel = Tensor::randn({1, n_mels, 3000}, DType::Float32, Device::GPU);
        }
        mel = mel.astype(dt);

        Tensor out;
        double best_ms = 1e30;
        for (int r = 0; r < std::max(repeat, 1); ++r) {
            t0 = std::chrono::steady_clock::now();
            out = enc.forward(mel);
            out.sync();
            backends::hip::synchronize();
            best_ms = std::min(best_ms, std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count());
        }
        Tensor host = out.cpu().astype(DType::Float32).ascontiguousarray();
        double sum = 0, sum_abs = 0;
        for (size_t i = 0; i < host.size(); ++i) {
            sum += host.typed_data<float>()[i];
            sum_abs += std::fabs(host.typed_data<float>()[i]);
        }
        if (!out_path.empty()) {
            std::ofstream f(out_path, std::ios::binary);
            f.write(reinterpret_cast<const char *>(host.typed_data<float>()), static_cast<std::streamsize>(host.size() * sizeof(float)));
        }
        printf("{\"d_model\": %zu, \"n_mels\": %zu, \"layers\": %d, \"heads\": %d, \"dtype\": \"%s\", \"frames\": %zu, \"out_shape\": [%zu, %zu, %zu], "
               "\"load_ms\": %.2f, \"forward_ms_best_of_%d\": %.3f, \"mean\": %.6g, \"mean_abs\": %.6g}\n",
               d_model, n_mels, layers, heads, dtype.c_str(), mel.shape()[2], host.shape()[0], host.shape()[1], host.shape()[2], load_ms, std::max(repeat, 1),
               best_ms, sum / double(host.size()), sum_abs / double(host.size()));
    } catch (const std::exception &e) {
        fprintf(stderr, "whisper_encoder: %s\n", e.what());
        return 1;
    }
    return 0;
}
