#pragma once
// Basic macros and helpers shared by the QuickMLP host code.

#define QUICKMLP_VERSION_MAJOR 0
#define QUICKMLP_VERSION_MINOR 1
#define QUICKMLP_VERSION_PATCH 0

#define QUICKMLP_NAMESPACE ::qmlp
#define QUICKMLP_NAMESPACE_BEGIN namespace qmlp {
#define QUICKMLP_NAMESPACE_END }

#include <cstdarg>
#include <cstdint>
#include <string>

// Forward declaration compatible with HIP's hipStream_t / hipEvent_t, so that public
// headers do not pull in the HIP runtime headers.
struct ihipStream_t;
struct ihipEvent_t;

QUICKMLP_NAMESPACE_BEGIN

typedef ihipStream_t* stream_t;
typedef ihipEvent_t* event_t;

// Host-side IEEE binary16 value (the storage type of the network parameters).
typedef _Float16 half;

class NonAssignable
{
public:
    NonAssignable(NonAssignable const&) = delete;
    NonAssignable& operator=(NonAssignable const&) = delete;
    NonAssignable() {}
};

/** Rounds 'numToRound' up to the next multiple of 'multiple'. */
template <typename T>
T roundUp(T numToRound, T multiple)
{
    return ((numToRound + multiple - 1) / multiple) * multiple;
}

template <typename T>
T divUp(T a, T b)
{
    return (a + b - 1) / b;
}

static inline void replaceAll(std::string& s, const std::string& search, const std::string& replace)
{
    if (search.empty()) return;
    for (size_t pos = 0;; pos += replace.length()) {
        pos = s.find(search, pos);
        if (pos == std::string::npos) break;
        s.replace(pos, search.length(), replace);
    }
}

/** Integer power x**p. */
template <typename T>
T ipow(T x, unsigned int p)
{
    T r = 1;
    while (p) {
        if (p & 1u) r *= x;
        x *= x;
        p >>= 1;
    }
    return r;
}

/** printf-style formatting into a std::string. */
std::string format(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
std::string vformat(const char* fmt, va_list ap);

QUICKMLP_NAMESPACE_END
