#include "rg_mirror/common.h"

namespace refactor {

    std::string_view DataType::name() const noexcept {
        switch (internal) {
            case F32: return "F32";
            case U8: return "U8";
            case I8: return "I8";
            case U16: return "U16";
            case I16: return "I16";
            case I32: return "I32";
            case I64: return "I64";
            case String: return "String";
            case Bool: return "Bool";
            case FP16: return "FP16";
            case F64: return "F64";
            case U32: return "U32";
            case U64: return "U64";
            case Complex64: return "Complex64";
            case Complex128: return "Complex128";
            case BF16: return "BF16";
        }
        return "?";
    }

    bool DataType::isFloat() const noexcept {
        return internal == F32 || internal == F64 || internal == FP16 || internal == BF16;
    }

    bool DataType::isCpuNumberic() const noexcept {
        switch (internal) {
            case F32: case F64: case U8: case I8: case U16: case I16:
            case I32: case I64: case U32: case U64:
                return true;
            default:
                return false;
        }
    }

    size_t DataType::size() const noexcept {
        switch (internal) {
            case U8: case I8: case Bool: return 1;
            case U16: case I16: case FP16: case BF16: return 2;
            case F32: case I32: case U32: return 4;
            case F64: case I64: case U64: case Complex64: return 8;
            case Complex128: return 16;
            case String: return sizeof(std::string);
        }
        return 0;
    }

}// namespace refactor
