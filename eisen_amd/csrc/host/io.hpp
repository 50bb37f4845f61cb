// Host-side IO around the training step: the pre-tokenised u16 stream that feeds it and the weight
// files that leave it.  Byte formats follow the reference exactly.
#pragma once
#include <cstdint>
#include <cstdio>
#include <string>
#include <utility>
#include <vector>

#include "graph.hpp"

namespace eisen {

// Targets of masked positions (src/data/fim.rs:173 uses usize::MAX; on this side targets are int64).
constexpr int64_t kIgnoreIndex = -1;

// BinaryDataLoader (src/data/dataloader.rs:84-198) without fill-in-the-middle: a file of little-endian
// u16 token ids is cut into windows of seq_len+1 tokens, batch_size windows per batch;
// x = window[0..seq_len) as f32, targets = window[1..seq_len+1).
// The reference reads through a std::io::BufReader of 4 MiB and refills its token buffer with ONE
// read() of 100 batches' worth whenever fewer than one batch is buffered.  A BufReader read that
// finds bytes left in its buffer returns only those, so refills can be short; next_batch() gives up
// (returns false) when a refill still leaves less than one batch.  Both behaviours are kept.
class BinaryDataLoader {
public:
    BinaryDataLoader(const std::string& path, size_t seq_len, size_t batch_size);
    ~BinaryDataLoader();
    BinaryDataLoader(const BinaryDataLoader&) = delete;
    BinaryDataLoader& operator=(const BinaryDataLoader&) = delete;

    size_t total_batches() const { return total_batches_; }
    size_t seq_len() const { return seq_len_; }
    size_t batch_size() const { return batch_size_; }
    // Fills x [batch*seq] and targets [batch*seq]; false when the stream is exhausted.
    bool next_batch(float* x, int64_t* targets);
    void reset();

private:
    size_t buffered_read(uint8_t* dst, size_t want);  // std::io::BufReader::read
    FILE* file_ = nullptr;
    size_t seq_len_, batch_size_, total_batches_ = 0;
    std::vector<uint16_t> buffer_;      // decoded tokens not yet handed out
    std::vector<uint8_t> rd_;           // the BufReader's buffer
    size_t rd_pos_ = 0, rd_len_ = 0;
    static constexpr size_t kReaderCapacity = 4 * 1024 * 1024;
};

// save_weights (examples/train_llm.rs:93-105): every parameter tensor in tensor-id order, f32 LE, no header.
void save_weights(Graph& g, const std::string& path);
// load_weights (examples/chat_cli.rs:161-180): consecutive f32 LE runs, one per id in `params`.
// Returns the number of floats consumed; throws when the file is too short.
size_t load_weights(Graph& g, const std::vector<size_t>& params, const std::string& path);
// write_safetensors (src/tools/huggingface.rs:88-146): F32 payload in `named` order, header sorted by
// name, 2-D tensors other than model.embed_tokens.weight transposed to [out, in].
void write_safetensors(Graph& g, const std::vector<std::pair<std::string, size_t>>& named, const std::string& path);

struct LlamaConfig {
    size_t vocab_size, hidden_size, intermediate_size, num_hidden_layers, num_attention_heads, num_key_value_heads,
        max_position_embeddings;
    float rms_norm_eps, rope_theta;
    bool tie_word_embeddings;
};
// write_llama_config (src/tools/huggingface.rs:38-84).  One deliberate difference: the reference
// prints num_attention_heads under "num_key_value_heads" as well, which describes a GQA model wrongly;
// here the real KV head count is written.
void write_llama_config(const std::string& path, const LlamaConfig& cfg);
// Rust's `{}` for an f32: shortest decimal that reads back to the same f32, never in exponent form.
std::string format_f32_display(float v);

}  // namespace eisen
