// Fail-fast helpers shared by the host runtime.
//
// The reference treats every error as fatal (blackriver/common.hpp:15-20,
// 53-81): a failed assertion or a non-OK operator return prints a message and
// aborts the process.  That stays the default here.  An embedding program may
// install a panic hook (set_panic_hook) that throws instead, which is how the
// C embedding API reports errors to its caller without killing it.
#pragma once

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <stdexcept>
#include <string>
#include <vector>

namespace br {

struct Panic : public std::runtime_error {
    explicit Panic(const std::string& what) : std::runtime_error(what) {}
};

using PanicHook = void (*)(const std::string& message);  // must not return
void set_panic_hook(PanicHook hook);
[[noreturn]] void panic_at(const char* file, int line, const std::string& msg);
void assert_at(const char* expr, bool ok, const char* file, int line, const char* msg);

// Device-runtime failures are fatal too (reference: COMPLAIN_ERROR_AND_EXIT).
void hip_check_at(const char* what, int code, const char* file, int line);

// read_data: a raw little-endian file read in blocks of 1024 elements; the
// element count must be a multiple of 1024 (blackriver/common.hpp:83-101).
template <typename T>
inline void read_data(const char* fileName, std::vector<T>& out);

}  // namespace br

#define br_assert(Expr, Msg) ::br::assert_at(#Expr, static_cast<bool>(Expr), __FILE__, __LINE__, Msg)
#define br_panic(Msg) ::br::panic_at(__FILE__, __LINE__, Msg)
#define BR_HIP_CHECK(call) ::br::hip_check_at(#call, (call), __FILE__, __LINE__)

// Same contract as the reference's op_check (common.hpp:59-63): panic on a
// non-OK operator result, otherwise return it.
#define op_check(ret, Msg)                          \
    if ((ret) != ::br::OP_OK) {                     \
        ::br::panic_at(__FILE__, __LINE__, Msg);    \
    }                                               \
    return ret

namespace br {

template <typename T>
inline void read_data(const char* fileName, std::vector<T>& out) {
    std::ifstream in(fileName, std::ios::binary | std::ios::ate);
    if (!in) panic_at(__FILE__, __LINE__, std::string("can't open file: ") + fileName);
    const size_t bytes = static_cast<size_t>(in.tellg());
    in.seekg(0, std::ios::beg);
    constexpr size_t kBlock = 1024;
    const size_t items = bytes / sizeof(T);
    br_assert(items % kBlock == 0, "Only support block read");
    out.resize(items);
    for (size_t done = 0; done < items; done += kBlock)
        in.read(reinterpret_cast<char*>(out.data() + done), sizeof(T) * kBlock);
}

}  // namespace br
