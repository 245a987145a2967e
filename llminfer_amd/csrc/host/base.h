// Host-side vocabulary of the engine this backend plugs into: status codes,
// device/data type enums, fatal-error macros.
// Mirrors code/include/base/base.h of the reference (enums :18-69, Status
// :103-137) with DeviceHIP taking the numeric slot DeviceCUDA had (:44-48).
// Where the reference aborts through glog (CHECK / LOG(FATAL)), this layer
// throws base::FatalError carrying file:line; uncaught, it terminates the
// process just the same.
#ifndef LLMI_HOST_BASE_H
#define LLMI_HOST_BASE_H

#include <cstddef>
#include <cstdint>
#include <sstream>
#include <stdexcept>
#include <string>

namespace model {
// The buffers on the attention path (base.h:25-29 keep the same numbers).
enum class ModelBufferType : uint8_t {
    TokenPosition = 1,
    SinCache = 3,
    CosCache = 4,
    Query = 6,
    KeyCache = 7,
    ValueCache = 8,
    KVSplitOutput = 9,
    MHAOutput = 10,
};
}  // namespace model

namespace base {

enum class DeviceType : uint8_t {
    DeviceUnknown = 0,
    DeviceHIP = 1,
    DeviceCPU = 2,
};

enum class DataType : uint8_t {
    DataTypeUnknown = 0,
    DataTypeFp32 = 1,
    DataTypeBf16 = 2,  // stored as uint16_t bit patterns
    DataTypeFp16 = 3,
    DataTypeInt32 = 4,
    DataTypeInt4x8 = 5,
};

class FatalError : public std::runtime_error {
public:
    explicit FatalError(const std::string& what) : std::runtime_error(what) {}
};

[[noreturn]] void fatal(const char* file, int line, const std::string& msg);

#define LLMI_FATAL(msg)                                  \
    do {                                                 \
        std::ostringstream llmi_oss_;                    \
        llmi_oss_ << msg;                                \
        ::base::fatal(__FILE__, __LINE__, llmi_oss_.str()); \
    } while (0)

#define LLMI_CHECK(cond)                                       \
    do {                                                       \
        if (!(cond)) LLMI_FATAL("Check failed: " #cond);       \
    } while (0)

size_t data_type_size(DataType data_type);  // base.h:78-87

class NoCopyable {
protected:
    NoCopyable() = default;
    ~NoCopyable() = default;
    NoCopyable(const NoCopyable&) = delete;
    NoCopyable& operator=(const NoCopyable&) = delete;
};

enum class StatusCode : uint8_t {
    Success = 0,
    FunctionUnImplement = 1,
    PathNotValid = 2,
    ModelParseError = 3,
    InternalError = 5,
    KeyValueHasExist = 6,
    InvalidArgument = 7,
};

class Status {
public:
    Status(StatusCode code = StatusCode::Success, std::string err_msg = "") : code_(code), err_msg_(std::move(err_msg)) {}
    Status& operator=(StatusCode code) {
        code_ = code;
        return *this;
    }
    bool operator==(StatusCode code) const { return code_ == code; }
    bool operator!=(StatusCode code) const { return code_ != code; }
    operator int() const { return static_cast<int>(code_); }
    operator bool() const { return code_ == StatusCode::Success; }
    StatusCode get_err_code() const { return code_; }
    const std::string& get_err_msg() const { return err_msg_; }
    void set_err_msg(const std::string& err_msg) { err_msg_ = err_msg; }

private:
    StatusCode code_;
    std::string err_msg_;
};

namespace error {
// STATUS_CHECK of the reference (base.h:127-137): a failed Status is fatal.
#define STATUS_CHECK(call)                                                                          \
    do {                                                                                            \
        const ::base::Status& llmi_status_ = (call);                                                \
        if (!llmi_status_)                                                                          \
            LLMI_FATAL("Infer error, code " << int(llmi_status_) << ": " << llmi_status_.get_err_msg()); \
    } while (0)

inline Status success(const std::string& m = "") { return Status(StatusCode::Success, m); }
inline Status function_not_implement(const std::string& m = "") { return Status(StatusCode::FunctionUnImplement, m); }
inline Status internal_error(const std::string& m = "") { return Status(StatusCode::InternalError, m); }
inline Status invalid_argument(const std::string& m = "") { return Status(StatusCode::InvalidArgument, m); }
}  // namespace error

}  // namespace base
#endif
