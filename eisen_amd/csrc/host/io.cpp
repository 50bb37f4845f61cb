#include "io.hpp"

#include <algorithm>
#include <cerrno>
#include <cmath>
#include <cstring>
#include <map>

namespace eisen {

namespace {
struct FileCloser {
    FILE* f;
    ~FileCloser() { if (f) fclose(f); }
};
void write_all(FILE* f, const void* p, size_t n, const std::string& path) {
    if (n && fwrite(p, 1, n, f) != n) throw Error("write to " + path + " failed: " + strerror(errno));
}
// host is little-endian (x86-64 / the GPU boxes); f32 and u64 go out as they lie in memory
static_assert(sizeof(float) == 4, "f32");
}  // namespace

// ---- BinaryDataLoader -----------------------------------------------------------------------

BinaryDataLoader::BinaryDataLoader(const std::string& path, size_t seq_len, size_t batch_size)
    : seq_len_(seq_len), batch_size_(batch_size), rd_(kReaderCapacity) {
    if (seq_len == 0 || batch_size == 0) throw Error("BinaryDataLoader: seq_len and batch_size must be positive");
    file_ = fopen(path.c_str(), "rb");
    if (!file_) throw Error("Binary file not found: " + path);
    setvbuf(file_, nullptr, _IONBF, 0);  // the buffering that matters is emulated below
    if (fseek(file_, 0, SEEK_END) != 0) throw Error("BinaryDataLoader: cannot seek " + path);
    const long size = ftell(file_);
    fseek(file_, 0, SEEK_SET);
    const size_t total_tokens = (size_t)size / 2;
    total_batches_ = total_tokens / (batch_size * (seq_len + 1));  // dataloader.rs:100-104
}

BinaryDataLoader::~BinaryDataLoader() {
    if (file_) fclose(file_);
}

// std::io::BufReader<File>::read: an empty buffer and a request at least as large as the buffer go
// straight to the file; otherwise the buffer is (re)filled with one read and as much of it as fits
// is handed out, even if that is less than was asked for.
size_t BinaryDataLoader::buffered_read(uint8_t* dst, size_t want) {
    if (rd_pos_ == rd_len_ && want >= kReaderCapacity) return fread(dst, 1, want, file_);
    if (rd_pos_ == rd_len_) {
        rd_len_ = fread(rd_.data(), 1, kReaderCapacity, file_);
        rd_pos_ = 0;
    }
    const size_t n = std::min(want, rd_len_ - rd_pos_);
    memcpy(dst, rd_.data() + rd_pos_, n);
    rd_pos_ += n;
    return n;
}

bool BinaryDataLoader::next_batch(float* x, int64_t* targets) {
    const size_t need = batch_size_ * (seq_len_ + 1);  // dataloader.rs:134
    if (buffer_.size() < need) {
        const size_t fetch = need * 100;
        std::vector<uint8_t> bytes(fetch * 2);
        const size_t got = buffered_read(bytes.data(), bytes.size());
        if (got == 0 && buffer_.size() < need) return false;
        const size_t old = buffer_.size();
        buffer_.resize(old + got / 2);  // chunks_exact(2): an odd trailing byte is dropped
        for (size_t i = 0; i < got / 2; i++) buffer_[old + i] = (uint16_t)(bytes[2 * i] | (bytes[2 * i + 1] << 8));
    }
    if (buffer_.size() < need) return false;
    for (size_t b = 0; b < batch_size_; b++) {
        const uint16_t* w = buffer_.data() + b * (seq_len_ + 1);
        for (size_t s = 0; s < seq_len_; s++) {
            x[b * seq_len_ + s] = (float)w[s];
            targets[b * seq_len_ + s] = (int64_t)w[s + 1];
        }
    }
    buffer_.erase(buffer_.begin(), buffer_.begin() + need);
    return true;
}

void BinaryDataLoader::reset() {  // dataloader.rs:200-203
    fseek(file_, 0, SEEK_SET);
    rd_pos_ = rd_len_ = 0;  // a BufReader seek discards its buffer
    buffer_.clear();
}

// ---- checkpoints ------------------------------------------------------------------------------

void save_weights(Graph& g, const std::string& path) {
    FILE* f = fopen(path.c_str(), "wb");
    if (!f) throw Error("Cannot create checkpoint file " + path + ": " + strerror(errno));
    FileCloser fc{f};
    for (size_t i = 0; i < g.num_params; i++) {
        const std::vector<float> data = g.sync_to_cpu(i);
        write_all(f, data.data(), data.size() * sizeof(float), path);
    }
    if (fflush(f) != 0) throw Error("flush of " + path + " failed");
}

size_t load_weights(Graph& g, const std::vector<size_t>& params, const std::string& path) {
    FILE* f = fopen(path.c_str(), "rb");
    if (!f) throw Error("Could not find model weights: " + path);
    FileCloser fc{f};
    fseek(f, 0, SEEK_END);
    const size_t floats = (size_t)ftell(f) / 4;  // chunks_exact(4)
    fseek(f, 0, SEEK_SET);
    size_t offset = 0;
    std::vector<float> chunk;
    for (size_t id : params) {
        const size_t n = g.at(id).size();
        if (offset + n > floats)
            throw Error("Weight file is truncated! Expected more than " + std::to_string(floats) + " floats [for sure " + std::to_string(offset + n) + "].");
        chunk.resize(n);
        if (n && fread(chunk.data(), sizeof(float), n, f) != n) throw Error("read of " + path + " failed");
        g.load_tensor_data(id, chunk.data(), n);
        offset += n;
    }
    return offset;
}

void write_safetensors(Graph& g, const std::vector<std::pair<std::string, size_t>>& named, const std::string& path) {
    struct Entry {
        std::vector<size_t> shape;
        size_t begin, end;
    };
    std::map<std::string, Entry> entries;  // BTreeMap<String, _>: byte-wise ascending names
    FILE* f = fopen(path.c_str(), "wb");
    if (!f) throw Error("Cannot create " + path + ": " + strerror(errno));
    FileCloser fc{f};

    // header first needs every offset, and offsets only need the sizes
    size_t cursor = 0;
    for (const auto& kv : named) {
        std::vector<size_t> shape = g.at(kv.second).shape;
        const size_t bytes = g.at(kv.second).size() * sizeof(float);
        if (shape.size() == 2 && kv.first != "model.embed_tokens.weight") std::swap(shape[0], shape[1]);
        entries[kv.first] = Entry{shape, cursor, cursor + bytes};  // a repeated name keeps the last one, like insert()
        cursor += bytes;
    }
    std::string header = "{";
    bool first = true;
    for (const auto& e : entries) {
        if (!first) header += ',';
        first = false;
        header += '"' + e.first + "\":{\"dtype\":\"F32\",\"shape\":[";
        for (size_t i = 0; i < e.second.shape.size(); i++) header += (i ? "," : "") + std::to_string(e.second.shape[i]);
        header += "],\"data_offsets\":[" + std::to_string(e.second.begin) + "," + std::to_string(e.second.end) + "]}";
    }
    header += '}';
    while (header.size() % 8 != 0) header += ' ';
    const uint64_t header_len = header.size();
    write_all(f, &header_len, 8, path);
    write_all(f, header.data(), header.size(), path);

    std::vector<float> t;
    for (const auto& kv : named) {
        const std::vector<float> data = g.sync_to_cpu(kv.second);
        const std::vector<size_t>& shape = g.at(kv.second).shape;
        if (shape.size() == 2 && kv.first != "model.embed_tokens.weight") {
            // [in, out] -> [out, in] (huggingface.rs:24-32, :104-109)
            const size_t rows = shape[0], cols = shape[1];
            t.resize(data.size());
            for (size_t r = 0; r < rows; r++)
                for (size_t c = 0; c < cols; c++) t[c * rows + r] = data[r * cols + c];
            write_all(f, t.data(), t.size() * sizeof(float), path);
        } else {
            write_all(f, data.data(), data.size() * sizeof(float), path);
        }
    }
    if (fflush(f) != 0) throw Error("flush of " + path + " failed");
}

std::string format_f32_display(float v) {
    if (std::isnan(v)) return "NaN";
    if (std::isinf(v)) return v < 0 ? "-inf" : "inf";
    char buf[64];
    int prec = 1;
    for (; prec <= 9; prec++) {  // shortest digit string that reads back to the same f32
        snprintf(buf, sizeof(buf), "%.*e", prec - 1, (double)v);
        if (strtof(buf, nullptr) == v) break;
    }
    // buf = d.ddddde[+-]xx  ->  plain decimal
    std::string s(buf);
    const size_t epos = s.find('e');
    const int exp10 = atoi(s.c_str() + epos + 1);
    std::string mant = s.substr(0, epos);
    bool neg = false;
    if (!mant.empty() && mant[0] == '-') { neg = true; mant.erase(0, 1); }
    std::string digits;
    for (char ch : mant) if (ch != '.') digits += ch;
    while (digits.size() > 1 && digits.back() == '0') digits.pop_back();
    std::string out;
    const int point = exp10 + 1;  // digits before the decimal point
    if (point <= 0) {
        out = "0." + std::string((size_t)(-point), '0') + digits;
    } else if ((size_t)point >= digits.size()) {
        out = digits + std::string((size_t)point - digits.size(), '0');
    } else {
        out = digits.substr(0, (size_t)point) + "." + digits.substr((size_t)point);
    }
    if (digits == "0") out = "0";
    return (neg ? "-" : "") + out;
}

void write_llama_config(const std::string& path, const LlamaConfig& c) {
    FILE* f = fopen(path.c_str(), "wb");
    if (!f) throw Error("Cannot create " + path + ": " + strerror(errno));
    FileCloser fc{f};
    std::string b = "{\n";
    b += "  \"architectures\": [\"LlamaForCausalLM\"],\n";
    b += "  \"model_type\": \"llama\",\n";
    b += "  \"vocab_size\": " + std::to_string(c.vocab_size) + ",\n";
    b += "  \"hidden_size\": " + std::to_string(c.hidden_size) + ",\n";
    b += "  \"intermediate_size\": " + std::to_string(c.intermediate_size) + ",\n";
    b += "  \"num_hidden_layers\": " + std::to_string(c.num_hidden_layers) + ",\n";
    b += "  \"num_attention_heads\": " + std::to_string(c.num_attention_heads) + ",\n";
    b += "  \"num_key_value_heads\": " + std::to_string(c.num_key_value_heads) + ",\n";
    b += "  \"max_position_embeddings\": " + std::to_string(c.max_position_embeddings) + ",\n";
    b += "  \"rms_norm_eps\": " + format_f32_display(c.rms_norm_eps) + ",\n";
    b += "  \"rope_theta\": " + format_f32_display(c.rope_theta) + ",\n";
    b += "  \"bos_token_id\": 1,\n  \"eos_token_id\": 2,\n  \"pad_token_id\": 0,\n  \"hidden_act\": \"silu\",\n";
    b += std::string("  \"tie_word_embeddings\": ") + (c.tie_word_embeddings ? "true" : "false") + ",\n";
    b += "  \"initializer_range\": 0.02,\n  \"torch_dtype\": \"float32\"\n}\n";
    write_all(f, b.data(), b.size(), path);
}

}  // namespace eisen
