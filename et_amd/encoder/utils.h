// Host-side utilities of the encoder layer: error check and the owning device
// array.  Mirrors encoder/utils.h of the reference (cudaChk -> etChk,
// Weight<T>) on top of the C ABI in et_amd.h, so this header needs no HIP
// headers.
#pragma once
#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <string>

#include "../../include/et_amd.h"

#if defined(__clang__) || (defined(__GNUC__) && __GNUC__ >= 12)
typedef _Float16 half;
#else
struct half {
    unsigned short bits;
};
#endif

// What a failed call does.  Default: print and exit(1), exactly like the
// reference's cudaChk (encoder/utils.h:6-12).  A host that prefers exceptions
// (the C wrappers used by the Python binding do) flips et_throw_on_error().
inline bool &et_throw_on_error() {
    static bool flag = false;
    return flag;
}

#define etChk(stat) etErrCheck_((stat), __FILE__, __LINE__)

inline void etErrCheck_(int stat, const char *file, int line) {
    if (stat >= 0)
        return;
    std::string msg = std::string("ET Error: ") + et_strerror(stat) + " (" + et_last_error() + ") " +
                      file + " " + std::to_string(line);
    if (et_throw_on_error())
        throw std::runtime_error(msg);
    fprintf(stderr, "%s\n", msg.c_str());
    exit(1);
}

// Precondition check with the same failure policy (the reference uses assert,
// e.g. encoder/encoder.cu:17).
inline void etRequire(bool ok, const char *what) {
    if (ok)
        return;
    std::string msg = std::string("ET Error: ") + what;
    if (et_throw_on_error())
        throw std::runtime_error(msg);
    fprintf(stderr, "%s\n", msg.c_str());
    exit(1);
}

// Move-only owning device array (encoder/utils.h:14-43).
template <typename T> class Weight {
    T *data;
    int size;

  public:
    explicit Weight(int size_) : data(nullptr), size(size_) {
        etChk(et_malloc(reinterpret_cast<void **>(&data), sizeof(T) * (size_t)size));
    }
    // copies `size_` elements from HOST memory
    Weight(const T *data_, int size_) : data(nullptr), size(size_) {
        etChk(et_malloc(reinterpret_cast<void **>(&data), sizeof(T) * (size_t)size));
        etChk(et_memcpy_h2d(data, data_, sizeof(T) * (size_t)size));
    }
    Weight() : data(nullptr), size(0) {}
    ~Weight() {
        if (data)
            et_free(data);
    }
    Weight(const Weight &) = delete;
    Weight &operator=(const Weight &) = delete;
    Weight(Weight &&w) noexcept : data(w.data), size(w.size) {
        w.data = nullptr;
        w.size = 0;
    }
    Weight &operator=(Weight &&w) noexcept {
        if (this != &w) {
            if (data)
                et_free(data);
            data = w.data;
            size = w.size;
            w.data = nullptr;
            w.size = 0;
        }
        return *this;
    }
    T *get() const { return data; }
    int count() const { return size; }
    void alloc(int n) {
        if (data)
            et_free(data);
        size = n;
        etChk(et_malloc(reinterpret_cast<void **>(&data), sizeof(T) * (size_t)n));
    }
    void set(const T *src) { etChk(et_memcpy_h2d(data, src, sizeof(T) * (size_t)size)); }
};
