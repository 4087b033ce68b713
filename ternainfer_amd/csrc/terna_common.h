// Shared device-side definitions for the TernaSpMM kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

namespace terna {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(16))) int i32x16;
typedef __attribute__((ext_vector_type(4))) int i32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr int kWave = 64;

// Which scaling rule the epilogue applies; each follows one reference source.
enum EpilogueKind : int {
    EP_I8_DECODE  = 0,  // bf16((float(acc) / s[m]) * ws[g])           Reduction_Kernel.cuh:45-60
    EP_I8_PREFILL = 1,  // bf16(float(acc) * (ws[g] / s[m])), 0 if s==0  epilogue_visitor_scale_ws.h:135-205
    EP_BF16       = 2,  // bf16(acc * scale[g]), fp32 scale             (bf16-activation family)
};

// What a kernel needs to check that a cached P2 copy still belongs to the reference-format tensors it was made from:
// the tensors as the caller passes them now, the fingerprint recorded when the copy was made, the copy's id and the
// host-visible words in which a mismatch is reported (word 0: any report; word 1 + id % 1023: the id).
// `total_bits` is the length of the sign stream when the copy was made: the check compares it with the length the
// caller's offset array states now before it samples the stream, so no sample lies past the end of a shorter stream
// that has taken the old one's place.
struct RepackGuard {
    const uint64_t* bitmap;
    const int* tile_off;
    const uint32_t* sign_words;
    const unsigned long long* expect;
    uint32_t* stale;
    int tiles;                       // N * K / 4096
    int total_bits;                  // sign bits (padded per tile) of the matrix the copy was made from
    uint32_t id;
};

// How quant_input (model.py:120-123) is evaluated.  The reference's two lines leave the intermediate precision to
// PyTorch, and its two ways of running them differ.  (`127 / tensor` there is Tensor.__rtruediv__, which PyTorch
// evaluates as tensor.reciprocal() * 127.)
//   QUANT_ROUNDED   s = bf16(127 / max(max|x|, 1e-5)); q = rint(fp32(x * s)) with that ROUNDED s -- the quantiser and
//                   the epilogue's division then use the same number (this library's default);
//   QUANT_COMPILED  what the @torch.compile'd method computes (one fused fp32 kernel, no intermediate rounding to
//                   bf16): q = rint(fp32(x * t)) with the UNROUNDED t = fp32(fp32(1 / max(max|x|, 1e-5)) * 127); the
//                   returned s is bf16(t);
//   QUANT_EAGER     what the same lines give without torch.compile on bf16 tensors: every op rounds to bf16 --
//                   s = bf16(bf16(1 / max(max|x|, bf16(1e-5))) * 127), q = rint(bf16(x * s)).
// In every mode the s that is published (and that the epilogue divides by) is the bf16 value.
enum QuantMode : int { QUANT_ROUNDED = 0, QUANT_COMPILED = 1, QUANT_EAGER = 2 };

struct Epilogue {
    const uint16_t* s;      // bf16 [M]       (int8 family)
    const uint16_t* ws;     // bf16 [ws_num]  (int8 family)
    const float*    scale;  // fp32 [ws_num]  (bf16 family)
    int             ws_num;
    int             kind;
};

__device__ __forceinline__ float bf16_bits_to_float(uint16_t h)
{
    return __uint_as_float(static_cast<uint32_t>(h) << 16);
}

// Round to nearest even (the rounding of __float2bfloat16_rn): gfx950's v_cvt_pk_bf16_f32.
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f)
{
    return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}
// Two at once: lo in bits 0..15, hi in bits 16..31 (one instruction).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi)
{
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}

// The per-row scale of quant_input from the row's max |x|: `s_bits` is what is published, the return value what
// multiplies the activations.
__device__ __forceinline__ float quant_scale(float amax, int mode, uint16_t* s_bits)
{
    const float floor_v = mode == QUANT_EAGER ? 1.0013580322265625e-05f /* bf16(1e-5) */ : 1e-5f;
    const float a = fmaxf(amax, floor_v);
    float t;
    if (mode == QUANT_ROUNDED) {
        t = __fdiv_rn(127.0f, a);
    } else {
        float r = __fdiv_rn(1.0f, a);
        if (mode == QUANT_EAGER) r = bf16_bits_to_float(float_to_bf16_bits(r));
        t = __fmul_rn(r, 127.0f);
    }
    *s_bits = float_to_bf16_bits(t);
    return mode == QUANT_COMPILED ? t : bf16_bits_to_float(*s_bits);
}
// One activation: clamp(rint(x * s_mul)), the product rounded to bf16 first in QUANT_EAGER.  Returned as a float in
// [-128, 127].
__device__ __forceinline__ float quant_value(float x, float s_mul, int mode)
{
    float p = __fmul_rn(x, s_mul);
    if (mode == QUANT_EAGER) p = bf16_bits_to_float(float_to_bf16_bits(p));
    return __builtin_amdgcn_fmed3f(rintf(p), -128.0f, 127.0f);
}

// Weight-scale group of output column n on the decode path (Reduction_Kernel.cuh:46-54).
__device__ __forceinline__ int ws_group_decode(int n, int N, int ws_num)
{
    if (ws_num == 3 && N == 3840) return n < 2560 ? 0 : (n < 3200 ? 1 : 2);
    return n / (N / ws_num);
}

// Decode rule for four consecutive columns n0 .. n0+3 with one integer division instead of four: a group is
// at least 16 columns wide (N >= 64, ws_num <= 4), so at most one group boundary falls inside the four.
__device__ __forceinline__ void ws_group_decode4(int n0, int N, int ws_num, int g[4])
{
    if (ws_num == 3 && N == 3840) {
#pragma unroll
        for (int v = 0; v < 4; ++v) g[v] = n0 + v < 2560 ? 0 : (n0 + v < 3200 ? 1 : 2);
        return;
    }
    const int q = N / ws_num;                   // uniform
    g[0] = n0 / q;
    const int next = (g[0] + 1) * q;            // first column of the next group
#pragma unroll
    for (int v = 1; v < 4; ++v) g[v] = g[0] + (n0 + v >= next ? 1 : 0);
}

// Prefill path: the group of the first column of the 128-wide tile that holds n, clamped
// (epilogue_visitor_scale_ws.h:135-148).
__device__ __forceinline__ int ws_group_prefill(int n, int N, int ws_num)
{
    const int c0 = n & ~127;
    int g;
    if (N == 3840) g = c0 < 2560 ? 0 : (c0 < 3200 ? 1 : 2);
    else g = c0 / (N / ws_num);
    return g < ws_num ? g : ws_num - 1;
}

// Scale factors of one output row m and four consecutive output columns n0..n0+3, fetched
// ahead of the main loop so that no global load sits between the last MFMA and the store.
struct EpilogueRegs {
    float s;        // activation scale of row m (int8 family)
    float w[4];     // weight-group scale of each column (bf16 family: the fp32 scale)
};

// Raw buffer loads: a resource (base, byte range) in scalar registers, a per-lane byte offset and a scalar offset.  A lane
// whose offset lies past the range gets zeros and touches no memory -- no clamped address, no masked branch.
constexpr int kBufferRsrcFlags = 0x00020000;                    // raw buffer, 32-bit data format
constexpr int kBufferOutOfRange = static_cast<int>(0x80000000u);   // a lane offset no buffer reaches

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_raw_buffer(const void* base, uint32_t bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), kBufferRsrcFlags);
}

// Makes the value live in registers at this point of the program: a load that produced it cannot be sunk
// past here (into a branch, next to its use), and is waited for here.
__device__ __forceinline__ void pin_registers(u32x4& v)
{
    asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w));
}

__device__ __forceinline__ void pin_registers(u32x2& v) { asm volatile("" : "+v"(v.x), "+v"(v.y)); }
__device__ __forceinline__ void pin_registers(f32x4& v) { asm volatile("" : "+v"(v.x), "+v"(v.y), "+v"(v.z), "+v"(v.w)); }
__device__ __forceinline__ void pin_registers(float2& v) { asm volatile("" : "+v"(v.x), "+v"(v.y)); }

// max / sum over the four lanes L, L ^ 16, L ^ 32, L ^ 48 with the row-swap permutations of the VALU (gfx950):
// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of its second,
// v_permlane32_swap the upper half of the first with the lower half of the second; applied to two copies of v, every
// lane ends up holding its own value and its partner's.  No LDS round trip; the order of the additions is the same in
// all four lanes.  (asm statements: through the builtins the compiler took the two results of a swap for equal.)
template <bool IS_MAX>
__device__ __forceinline__ float cross_row_reduce(float v)
{
    auto op = [](float a, float b) { return IS_MAX ? fmaxf(a, b) : a + b; };
    float a = v, b = v;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    v = op(a, b);
    a = v;
    b = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
    return op(a, b);
}

// Compile-time loop: the body receives the index as a constant, so register arrays indexed by it
// never need dynamic addressing.
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

// Weight-group scales of the four consecutive output columns n0..n0+3.
__device__ __forceinline__ void load_col_scales(const Epilogue& ep, int n0, int N, float w[4])
{
    if (ep.ws_num == 1) {                       // one scale per matrix: no group arithmetic
        const float v = ep.kind == EP_BF16 ? ep.scale[0] : bf16_bits_to_float(ep.ws[0]);
        w[0] = w[1] = w[2] = w[3] = v;
        return;
    }
    int gd[4];
    ws_group_decode4(n0, N, ep.ws_num, gd);
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int g = ep.kind == EP_I8_PREFILL ? ws_group_prefill(n0 + v, N, ep.ws_num) : gd[v];
        w[v] = ep.kind == EP_BF16 ? ep.scale[g] : bf16_bits_to_float(ep.ws[g]);
    }
}

__device__ __forceinline__ EpilogueRegs load_epilogue(const Epilogue& ep, int m, int n0, int N)
{
    EpilogueRegs r;
    r.s = ep.kind == EP_BF16 ? 1.0f : bf16_bits_to_float(ep.s[m]);
    load_col_scales(ep, n0, N, r.w);
    return r;
}

// The same scale factors as they come out of memory -- bf16 storage (int8 family) or fp32 bits (bf16
// family) -- with no arithmetic on them: a kernel that requests them ahead of its main loop must not
// touch the values before the loop is over, or it waits for them (and for every load issued before
// them) on the spot.  finish_epilogue() converts once the data is certainly there.
struct EpilogueRaw {
    uint32_t s;
    uint32_t w[4];
};

__device__ __forceinline__ EpilogueRaw load_epilogue_raw(const Epilogue& ep, int m, int n0, int N)
{
    EpilogueRaw r;
    r.s = 0u;
    r.w[0] = r.w[1] = r.w[2] = r.w[3] = 0u;
    if (ep.kind == EP_BF16) {
        if (ep.ws_num == 1) {
            r.w[0] = __float_as_uint(ep.scale[0]);
        } else {
            int gd[4];
            ws_group_decode4(n0, N, ep.ws_num, gd);
#pragma unroll
            for (int v = 0; v < 4; ++v) r.w[v] = __float_as_uint(ep.scale[gd[v]]);
        }
    } else {
        r.s = ep.s[m];
        if (ep.ws_num == 1) {
            r.w[0] = ep.ws[0];
        } else {
            int gd[4];
            ws_group_decode4(n0, N, ep.ws_num, gd);
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int g = ep.kind == EP_I8_PREFILL ? ws_group_prefill(n0 + v, N, ep.ws_num) : gd[v];
                r.w[v] = ep.ws[g];
            }
        }
    }
    return r;
}

// The same without a load inside a branch (the compiler waits for every outstanding load at the join behind one):
// the group indices are computed first (arithmetic only) and all five values are loaded unconditionally; with one
// scale per matrix the four weight-scale loads read the same word.  F32 = the bf16-activation family.  Measured: this
// form is the faster one where the loads sit in a chain of dependent round trips (reference-format kernel, +4 %), the
// branching form where they follow a burst of independent loads (P2 kernel, +3 %).
template <bool F32>
__device__ __forceinline__ EpilogueRaw load_epilogue_raw_flat(const Epilogue& ep, int m, int n0, int N)
{
    EpilogueRaw r;
    int gd[4] = {0, 0, 0, 0};
    if (ep.ws_num != 1) ws_group_decode4(n0, N, ep.ws_num, gd);
    if constexpr (F32) {
        r.s = 0u;
#pragma unroll
        for (int v = 0; v < 4; ++v) r.w[v] = __float_as_uint(ep.scale[gd[v]]);
    } else {
        int g[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int gp = ep.ws_num != 1 ? ws_group_prefill(n0 + v, N, ep.ws_num) : 0;
            g[v] = ep.kind == EP_I8_PREFILL ? gp : gd[v];
        }
        r.s = ep.s[m];
#pragma unroll
        for (int v = 0; v < 4; ++v) r.w[v] = ep.ws[g[v]];
    }
    return r;
}

// Only the weight-group scales (the caller has the activation scale from elsewhere).
__device__ __forceinline__ EpilogueRaw load_epilogue_raw_scales(const Epilogue& ep, int n0, int N)
{
    EpilogueRaw r;
    r.s = 0u;
    int gd[4] = {0, 0, 0, 0};
    if (ep.ws_num != 1) ws_group_decode4(n0, N, ep.ws_num, gd);
#pragma unroll
    for (int v = 0; v < 4; ++v) r.w[v] = ep.ws[gd[v]];       // unconditional: see load_epilogue_raw
    return r;
}

__device__ __forceinline__ EpilogueRegs finish_epilogue(const Epilogue& ep, const EpilogueRaw& r)
{
    EpilogueRegs e;
    const bool f32 = ep.kind == EP_BF16;
    e.s = f32 ? 1.0f : __uint_as_float(r.s << 16);
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const uint32_t bits = r.w[ep.ws_num == 1 ? 0 : v];
        e.w[v] = f32 ? __uint_as_float(bits) : __uint_as_float(bits << 16);
    }
    return e;
}

// One output element: integer or float accumulator -> bf16 storage.
template <typename Acc>
__device__ __forceinline__ uint16_t apply_epilogue(int kind, const EpilogueRegs& e, int v, Acc acc)
{
    float r;
    if (kind == EP_BF16) {
        r = static_cast<float>(acc) * e.w[v];
    } else if (kind == EP_I8_DECODE) {
        r = __fmul_rn(__fdiv_rn(static_cast<float>(acc), e.s), e.w[v]);
    } else {
        const float coeff = (e.s != 0.0f) ? __fdiv_rn(e.w[v], e.s) : 0.0f;
        r = __fmul_rn(static_cast<float>(acc), coeff);
    }
    return float_to_bf16_bits(r);
}

// Expansion tables: index = (nonzero nibble << 4) | (next 4 sign bits of the stream).
// The j-th set bit of the nibble takes sign bit number popcount(nibble below j).
//   bf16 table: 4 x bf16 (+1 = 0x3F80, -1 = 0xBF80) in 8 bytes
//   int8 table: 4 x int8 (+1 = 0x01,  -1 = 0xFF)   in 4 bytes
__device__ __forceinline__ uint2 make_lut_bf16(int e)
{
    const int nz = e >> 4, sg = e & 15;
    uint32_t v[4];
    int used = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if ((nz >> j) & 1) {
            v[j] = ((sg >> used) & 1) ? 0xBF80u : 0x3F80u;
            ++used;
        } else {
            v[j] = 0u;
        }
    }
    return make_uint2(v[0] | (v[1] << 16), v[2] | (v[3] << 16));
}

__device__ __forceinline__ uint32_t make_lut_i8(int e)
{
    const int nz = e >> 4, sg = e & 15;
    uint32_t r = 0;
    int used = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if ((nz >> j) & 1) {
            r |= (((sg >> used) & 1) ? 0xFFu : 0x01u) << (8 * j);
            ++used;
        }
    }
    return r;
}

}  // namespace terna
