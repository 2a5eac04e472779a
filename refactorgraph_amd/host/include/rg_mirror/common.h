// Boundary vocabulary shared by every layer of the host mirror: element types, small aliases
// and the error macros.  Restates what the kernel plugin surface of InfiniTensor/RefactorGraph
// needs from its 00common layer (src/00common/include/common/{data_type.h,error_handler.h},
// src/00common/include/common.h:17-25), without the fmt / abseil dependencies.
#pragma once

#include <cstddef>
#include <cstdint>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <string_view>
#include <vector>

namespace refactor {

    using dim_t = uint32_t;
    template<class T> using Arc = std::shared_ptr<T>;

    // Element type with the reference's (ONNX) codes, src/00common/include/common/data_type.h:19-36.
    struct DataType {
        enum : uint8_t {
            F32 = 1, U8 = 2, I8 = 3, U16 = 4, I16 = 5, I32 = 6, I64 = 7, String = 8, Bool = 9,
            FP16 = 10, F64 = 11, U32 = 12, U64 = 13, Complex64 = 14, Complex128 = 15, BF16 = 16,
        } internal;

        constexpr DataType(decltype(internal) i) noexcept : internal(i) {}
        constexpr operator decltype(internal)() const noexcept { return internal; }

        std::string_view name() const noexcept;
        bool isFloat() const noexcept;        // F32, F64, FP16, BF16
        bool isCpuNumberic() const noexcept;  // numeric types a plain CPU loop can compute in
        size_t size() const noexcept;
    };

    struct UnimplementError : public std::logic_error {
        using std::logic_error::logic_error;
    };
    struct UnreachableError : public std::logic_error {
        using std::logic_error::logic_error;
    };

    namespace detail {
        template<class... Args> std::string cat(Args const &...args) {
            std::ostringstream os;
            (os << ... << args);
            return os.str();
        }
        inline std::string located(std::string msg, char const *file, int line) {
            return cat(msg, " Source ", file, ':', line);
        }
    }// namespace detail

}// namespace refactor

// Same names and exception types as src/00common/include/common/error_handler.h:19-39; messages
// carry the same " Source file:line" suffix.
#define ERROR_MSG(MSG) ::refactor::detail::located((MSG), __FILE__, __LINE__)
#define RUNTIME_ERROR(MSG) throw std::runtime_error(ERROR_MSG(MSG))
#define TODO(MSG) throw ::refactor::UnimplementError(ERROR_MSG(MSG))
#define UNREACHABLEX(T, ...)                                                                                 \
    [&]() -> T {                                                                                             \
        throw ::refactor::UnreachableError(ERROR_MSG(::refactor::detail::cat("Unreachable: ", __VA_ARGS__))); \
    }()
#define UNREACHABLE() UNREACHABLEX(void, "no message")
#define ASSERT(CONDITION, ...)                                                                  \
    {                                                                                           \
        if (!(CONDITION)) RUNTIME_ERROR(::refactor::detail::cat("Assertion: ", __VA_ARGS__));  \
    }
