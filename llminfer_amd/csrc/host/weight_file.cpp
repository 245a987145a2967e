#include "weight_file.h"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdlib>
#include <cstring>

namespace model {

namespace {
base::Status path_not_valid(const std::string& m) { return base::Status(base::StatusCode::PathNotValid, m); }
base::Status parse_error(const std::string& m) { return base::Status(base::StatusCode::ModelParseError, m); }
}  // namespace

base::Status WeightFile::open(const std::string& path, std::unique_ptr<WeightFile>* out, int32_t header_ints) {
    if (!out) return base::error::invalid_argument("null output");
    if (header_ints != 7 && header_ints != 8) return base::error::invalid_argument("header_ints must be 7 or 8");
    if (path.empty())  // model.cpp:131-133
        return path_not_valid("Failed to open the weight file, the model path is empty!");
    const int fd = ::open(path.c_str(), O_RDONLY);
    if (fd == -1)  // :136-139
        return path_not_valid("Failed to open the weight file " + path + ", may be the path does not exist!");
    struct stat st;
    if (fstat(fd, &st) == -1) {  // :161-165
        ::close(fd);
        return parse_error("Failed to retrieve the file size information from the model file.");
    }
    const size_t file_size = static_cast<size_t>(st.st_size);
    const size_t header_bytes = sizeof(int32_t) * static_cast<size_t>(header_ints);
    if (file_size < header_bytes) {  // :148-150
        ::close(fd);
        return parse_error("Failed to retrieve the configuration information from the model file.");
    }
    void* map = mmap(nullptr, file_size, PROT_READ, MAP_PRIVATE, fd, 0);  // :167-170
    if (map == MAP_FAILED || map == nullptr) {
        ::close(fd);
        return parse_error("Failed to map the weight file " + path + " into memory.");
    }
    std::unique_ptr<WeightFile> f(new WeightFile());
    f->fd_ = fd;
    f->map_ = map;
    f->file_size_ = file_size;
    std::memcpy(&f->config_, map, header_bytes);  // immediate_dim stays 0 for the 7-int header
    f->payload_ = reinterpret_cast<const uint16_t*>(static_cast<const char*>(map) + header_bytes);  // :177
    f->payload_elems_ = (file_size - header_bytes) / sizeof(uint16_t);

    // (|INT32_MIN| does not exist: a header that says so is not a model)
    if (f->config_.vocab_size == INT32_MIN) return parse_error("The vocabulary size in the model file is out of range.");
    if (header_ints == 7) {  // header and raw payload only: that file predates the layout below
        f->vocab_size_ = std::abs(f->config_.vocab_size);
        *out = std::move(f);
        return base::error::success();
    }
    // Model::generate_model_info, model.cpp:210-236 (its CHECKs become a parse error here)
    const ModelConfig& c = f->config_;
    if (c.dim <= 0 || c.hidden_dim <= 0 || c.layer_num <= 0 || c.head_num <= 0 || c.kv_head_num <= 0 ||
        c.vocab_size == 0 || c.max_seq_len <= 0 || c.immediate_dim < 0)
        return parse_error("The configuration in the model file is not positive.");
    if (c.dim % c.head_num != 0) return parse_error("dim is not a multiple of head_num.");            // :221
    f->head_dim_ = c.dim / c.head_num;                                                                  // :222
    // The header is untrusted input: every product below is formed in 64 bits and checked.
    const int64_t kv_dim64 = static_cast<int64_t>(f->head_dim_) * c.kv_head_num;                       // :223
    if (kv_dim64 > INT32_MAX || static_cast<int64_t>(c.dim) + 2 * kv_dim64 > INT32_MAX)
        return parse_error("kv_dim in the model file is out of range.");
    f->kv_dim_ = static_cast<int32_t>(kv_dim64);
    if (f->head_dim_ % 2 != 0) return parse_error("head_dim is odd.");                                 // :224
    if (c.head_num % c.kv_head_num != 0) return parse_error("head_num is not a multiple of kv_head_num.");  // :226
    f->vocab_size_ = std::abs(c.vocab_size);                                                            // :233

    // The offset walk of qwen3_fused.cpp:246-314, in elements.
    const size_t L = static_cast<size_t>(c.layer_num), hid = static_cast<size_t>(c.hidden_dim);
    const size_t dim = static_cast<size_t>(c.dim), kv = static_cast<size_t>(f->kv_dim_);
    const size_t imm = static_cast<size_t>(c.immediate_dim), hd = static_cast<size_t>(f->head_dim_);
    // Every tensor has to fit the payload, so a term beyond it (or a product that wraps) ends the walk:
    // a crafted header cannot make the sum wrap round to the file size.
    size_t off = 0;
    bool fits = true;
    const size_t limit = f->payload_elems_;
    auto advance = [&](size_t a, size_t b, size_t c3) {
        size_t ab = 0, abc = 0;
        if (__builtin_mul_overflow(a, b, &ab) || __builtin_mul_overflow(ab, c3, &abc) || abc > limit || off > limit - abc) {
            fits = false;
            return;
        }
        off += abc;
    };
    f->off_embedding_ = off;  advance(static_cast<size_t>(f->vocab_size_), hid, 1);  // 1. embedding
    f->off_pre_norm_ = off;   advance(L, hid, 1);                                    // 2. pre-attention RMSNorm
    f->off_qkv_ = off;        advance(L, dim + 2 * kv, hid);                         // 3. packed QKV projection
    f->off_qk_norm_ = off;    advance(L, 2, hd);                                     // 4. q_norm, k_norm
    f->off_o_ = off;          advance(L, hid, dim);                                  // 5. output projection
    f->off_ffn_norm_ = off;   advance(L, hid, 1);                                    // 6. FFN RMSNorm
    f->off_gate_up_ = off;    advance(L, 2 * imm, hid);                              // 7. gate and up projections
    f->off_down_ = off;       advance(L, hid, imm);                                  // 8. down projection
    f->off_final_norm_ = off; advance(hid, 1, 1);                                    // 9. final RMSNorm
    f->total_elems_ = off;                                                           // 10. lm_head is the embedding
    if (!fits)
        return parse_error("The model file is " + std::to_string(file_size) + " bytes, shorter than the tensors its header describes.");
    if (header_bytes + off * sizeof(uint16_t) != file_size)  // :317-318
        return parse_error("The model file is " + std::to_string(file_size) + " bytes, its header describes " +
                           std::to_string(header_bytes + off * sizeof(uint16_t)) + ".");
    *out = std::move(f);
    return base::error::success();
}

WeightFile::~WeightFile() {
    if (map_) munmap(map_, file_size_);
    if (fd_ != -1) ::close(fd_);
}

size_t WeightFile::layer_off(size_t base_off, int32_t layer, size_t per_layer) const {
    LLMI_CHECK(layer >= 0 && layer < config_.layer_num);
    return base_off + static_cast<size_t>(layer) * per_layer;
}

const uint16_t* WeightFile::pre_rmsnorm(int32_t l) const { return weight_ptr(layer_off(off_pre_norm_, l, config_.hidden_dim)); }
const uint16_t* WeightFile::qkv_proj(int32_t l) const {
    return weight_ptr(layer_off(off_qkv_, l, static_cast<size_t>(config_.dim + 2 * kv_dim_) * config_.hidden_dim));
}
const uint16_t* WeightFile::qk_norm(int32_t l) const { return weight_ptr(layer_off(off_qk_norm_, l, 2 * static_cast<size_t>(head_dim_))); }
const uint16_t* WeightFile::o_proj(int32_t l) const {
    return weight_ptr(layer_off(off_o_, l, static_cast<size_t>(config_.hidden_dim) * config_.dim));
}
const uint16_t* WeightFile::ffn_rmsnorm(int32_t l) const { return weight_ptr(layer_off(off_ffn_norm_, l, config_.hidden_dim)); }
const uint16_t* WeightFile::gate_up(int32_t l) const {
    return weight_ptr(layer_off(off_gate_up_, l, 2 * static_cast<size_t>(config_.immediate_dim) * config_.hidden_dim));
}
const uint16_t* WeightFile::down_proj(int32_t l) const {
    return weight_ptr(layer_off(off_down_, l, static_cast<size_t>(config_.hidden_dim) * config_.immediate_dim));
}

}  // namespace model
