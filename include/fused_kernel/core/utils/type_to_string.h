// typeToString<T>(): the C++ spelling of a type as a string, for messages and file names.
// Interface counterpart: FK/core/utils/type_to_string.h:156-160 (the demangled typeid name).
#ifndef FK_AMD_TYPE_TO_STRING_H
#define FK_AMD_TYPE_TO_STRING_H
#include <cstdlib>
#include <string>
#include <typeinfo>
#include <cxxabi.h>
namespace fk {
template <typename T> inline std::string typeToString() {
    int status = 0;
    char* demangled = abi::__cxa_demangle(typeid(T).name(), nullptr, nullptr, &status);
    std::string name = (status == 0 && demangled) ? demangled : typeid(T).name();
    std::free(demangled);
    return name;
}
} // namespace fk
#endif
