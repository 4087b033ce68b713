// Host-side helpers shared by the translation units of libternaspmm.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <unordered_map>

namespace terna {

[[noreturn]] inline void die(const char* what, hipError_t e, int line)
{
    std::printf("Last Cuda Error Detected at line: %d, Error: %s (%s).\n", line, hipGetErrorString(e), what);
    std::fflush(stdout);
    std::exit(EXIT_FAILURE);
}

inline bool shape_ok(int M, int N, int K)
{
    if (M < 1 || N < 64 || K < 64 || (N % 64) || (K % 64)) {
        std::printf("TernaSpMM Error: unsupported shape M=%d N=%d K=%d (need M >= 1, N %% 64 == 0, K %% 64 == 0)\n",
                    M, N, K);
        std::fflush(stdout);
        return false;
    }
    return true;
}

// int8 activations on the P2 layout: the 32-bit accumulator holds 64 times the sum (packed_common.h), which bounds K
inline bool i8_depth_ok(int K)
{
    constexpr int kMaxK = (1 << 18) - 64;
    if (K > kMaxK) {
        std::printf("TernaSpMM Error: unsupported K=%d with int8 activations (need K <= %d)\n", K, kMaxK);
        std::fflush(stdout);
        return false;
    }
    return true;
}

// weight_scale has four slots (convert/convert_TernaInfer.py:176-194): one to four scale groups per matrix
inline bool groups_ok(int ws_num)
{
    if (ws_num < 1 || ws_num > 4) {
        std::printf("TernaSpMM Error: unsupported ws_num=%d (need 1 .. 4)\n", ws_num);
        std::fflush(stdout);
        return false;
    }
    return true;
}

// Tuning overrides (TERNASPMM_DECODE_WAVES, TERNASPMM_PREFILL_BM, ...) force one of the kernel variants the library
// otherwise picks by shape.  They are honoured only when TERNASPMM_TUNING=1 is set as well: a shipped library does not
// change kernels because a variable of that name happens to be in the environment.
inline const char* tuning_env(const char* name)
{
    static const bool on = [] {
        const char* v = std::getenv("TERNASPMM_TUNING");
        return v != nullptr && std::atoi(v) == 1;
    }();
    return on ? std::getenv(name) : nullptr;
}

// Dynamic-LDS opt-in of one kernel, once per (kernel, device) of the process: the attribute is per device.
inline void allow_dynamic_lds_ptr(const void* kernel, int bytes, const char* what, int line)
{
    static std::mutex mutex;
    static std::unordered_map<const void*, uint64_t> done;       // kernel -> bit per device ordinal
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = -1;
    std::lock_guard<std::mutex> lock(mutex);
    uint64_t& mask = done[kernel];
    if (dev >= 0 && ((mask >> dev) & 1u)) return;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) die(what, e, line);
    if (dev >= 0) mask |= uint64_t{1} << dev;
}
template <typename Kernel>
void allow_dynamic_lds(Kernel kernel, int bytes, const char* what, int line)
{
    allow_dynamic_lds_ptr(reinterpret_cast<const void*>(kernel), bytes, what, line);
}

// The process-wide quant_input mode (QuantMode in terna_common.h; ternaspmm_quant_mode sets it, TERNASPMM_QUANT_MODE in
// the environment gives the initial value).  Defined in ternaspmm.hip.
int quant_mode();

// Shapes the attention entry points accept (head sizes 64 and 128, whole kv groups, caches of up to 8192 slots).
inline bool attention_args_ok(const char* who, int B, int H, int KV, int D, int S)
{
    if (B < 1 || H < 1 || KV < 1 || H % KV != 0 || (D != 64 && D != 128) || S < 1 || S > 8192) {
        std::fprintf(stderr, "%s: unsupported arguments (H=%d KV=%d D=%d S=%d)\n", who, H, KV, D, S);
        return false;
    }
    return true;
}

}  // namespace terna
