// Names of types as text, for messages and generated code (host only).
//
// Follows the reference's core/utils/type_to_string.h:41-157 for this compiler family: typeToStringView<T>() cuts the
// name out of the compiler's own function signature at compile time; typeToString<T>() demangles typeid(T).name() and
// spells enumerator template arguments, which the demangler prints as C casts "(fk::ND)2", as static_cast<fk::ND>(2), so
// that the text is valid C++ again.
#ifndef FK_CORE_TYPE_TO_STRING_H
#define FK_CORE_TYPE_TO_STRING_H

#include <cctype>
#include <cstdlib>
#include <cxxabi.h>
#include <string>
#include <string_view>
#include <typeinfo>

namespace fk {
template <typename T>
constexpr std::string_view typeToStringView() {
    constexpr std::string_view signature = __PRETTY_FUNCTION__;
    constexpr std::string_view prefix = "[T = ";
    constexpr size_t begin = signature.find(prefix) + prefix.size();
    constexpr size_t end = signature.rfind(']');
    return signature.substr(begin, end - begin);
}

namespace detail {
inline std::string demangle_name(const char* mangled) {
    int status = 0;
    char* const text = abi::__cxa_demangle(mangled, nullptr, nullptr, &status);
    std::string out = (status == 0 && text != nullptr) ? text : mangled;
    std::free(text);
    return out;
}
inline bool names_a_type(const std::string& s) {
    if (s.empty() || !(std::isalpha(static_cast<unsigned char>(s[0])) || s[0] == '_')) return false;
    for (const char c : s) {
        if (!(std::isalnum(static_cast<unsigned char>(c)) || c == '_' || c == ':')) return false;
    }
    return true;
}
// "(Type)value" -> "static_cast<Type>(value)" wherever Type looks like a (qualified) identifier
inline std::string convert_c_casts_to_static_cast(const std::string& in) {
    std::string out;
    size_t pos = 0;
    while (pos < in.size()) {
        const size_t open = in.find('(', pos);
        if (open == std::string::npos) break;
        const size_t close = in.find(')', open + 1);
        if (close == std::string::npos) break;
        const std::string type = in.substr(open + 1, close - open - 1);
        size_t value_end = close + 1;
        while (value_end < in.size() && (std::isalnum(static_cast<unsigned char>(in[value_end])) || in[value_end] == '_')) ++value_end;
        if (names_a_type(type) && value_end > close + 1) {
            out += in.substr(pos, open - pos) + "static_cast<" + type + ">(" + in.substr(close + 1, value_end - close - 1) + ")";
            pos = value_end;
        } else {
            out += in.substr(pos, open + 1 - pos);
            pos = open + 1;
        }
    }
    return out + in.substr(pos);
}
} // namespace detail

template <typename T>
inline std::string typeToString() {
    return detail::convert_c_casts_to_static_cast(detail::demangle_name(typeid(T).name()));
}
} // namespace fk
#endif
