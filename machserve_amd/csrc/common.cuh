// Shared definitions of the gfx950 kernels: element type of this build, MFMA wrappers,
// wave reductions and the error channel of the extern "C" entry points.
//
// One library is built per element type: MS_ELEM_BF16 or MS_ELEM_F16 (bfloat16 or half-precision
// storage, 32-bit accumulation; MS_ELEM_HALF is defined for both: they share every tile and
// schedule) or MS_ELEM_F32 (everything in true 32-bit; its matrix products use the
// full-precision v_mfma_f32_16x16x4_f32, never a reduced-precision mode).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#if (defined(MS_ELEM_BF16) + defined(MS_ELEM_F16) + defined(MS_ELEM_F32)) != 1
#error "define exactly one of MS_ELEM_BF16, MS_ELEM_F16, MS_ELEM_F32"
#endif
#if defined(MS_ELEM_BF16) || defined(MS_ELEM_F16)
#define MS_ELEM_HALF 1
#endif

namespace ms {

constexpr int WAVE = 64;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// ---- element type ---------------------------------------------------------------
#if defined(MS_ELEM_BF16)
typedef __bf16 elem_t;
#elif defined(MS_ELEM_F16)
typedef _Float16 elem_t;
#else
typedef float elem_t;
#endif
// Half precision has five bits of exponent: a value of the 32-bit stream times a norm's weight, not yet divided by
// the row's root mean square, may lie outside its range (or among its subnormals), which bfloat16, with float's
// exponent, and float itself do not mind.  The forms that round such a value (the norm folded into the product
// that reads it) are not taken in the half-precision build: there the norm runs first and rounds after the division.
#if defined(MS_ELEM_F16)
constexpr bool kRoundsBeforeTheNormIsSafe = false;
#else
constexpr bool kRoundsBeforeTheNormIsSafe = true;
#endif
#ifdef MS_ELEM_HALF
constexpr bool kHalf = true;  // two-byte elements
typedef elem_t half8_t __attribute__((ext_vector_type(8)));
typedef elem_t half4_t __attribute__((ext_vector_type(4)));
#else
constexpr bool kHalf = false;
#endif

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(__bf16 v) { return (float)v; }
__device__ __forceinline__ float to_f32(_Float16 v) { return (float)v; }

// Round-to-nearest-even conversion of the compiler's own casts.
template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ __bf16 from_f32<__bf16>(float v) { return (__bf16)v; }
template <> __device__ __forceinline__ _Float16 from_f32<_Float16>(float v) { return (_Float16)v; }

// A fragment is 8 consecutive elements along the reduction dimension of one row of an
// operand: for lane l of a wave, row l % 16 and elements (l / 16) * 8 .. + 8 of a chunk of
// 32.  Both operands of a product use the same split, so the sum over the chunk is
// complete whatever order the hardware takes the elements in.
struct alignas(16) Frag {
#ifdef MS_ELEM_HALF
    half8_t v;
#else
    float v[8];
#endif
};

__device__ __forceinline__ Frag frag_zero() {
    Frag f;
#ifdef MS_ELEM_HALF
    for (int i = 0; i < 8; ++i) f.v[i] = (elem_t)0.0f;
#else
    for (int i = 0; i < 8; ++i) f.v[i] = 0.0f;
#endif
    return f;
}

// Load 8 consecutive elements (16-byte aligned for bf16, 32-byte for float).
__device__ __forceinline__ Frag frag_load(const elem_t* p) {
    Frag f;
#ifdef MS_ELEM_HALF
    f.v = *reinterpret_cast<const half8_t*>(p);
#else
    const f32x4* q = reinterpret_cast<const f32x4*>(p);
    f32x4 a = q[0], b = q[1];
    f.v[0] = a[0]; f.v[1] = a[1]; f.v[2] = a[2]; f.v[3] = a[3];
    f.v[4] = b[0]; f.v[5] = b[1]; f.v[6] = b[2]; f.v[7] = b[3];
#endif
    return f;
}

__device__ __forceinline__ void frag_store(elem_t* p, const Frag& f) {
#ifdef MS_ELEM_HALF
    *reinterpret_cast<half8_t*>(p) = f.v;
#else
    f32x4* q = reinterpret_cast<f32x4*>(p);
    f32x4 a = {f.v[0], f.v[1], f.v[2], f.v[3]}, b = {f.v[4], f.v[5], f.v[6], f.v[7]};
    q[0] = a; q[1] = b;
#endif
}

// acc[16x16] += A[16 rows x 32] * B[16 cols x 32]^T, both given as fragments.
// Result layout: lane l holds rows (l / 16) * 4 + i (i = 0..3) of column l % 16.
__device__ __forceinline__ void mma_16x16x32(f32x4& acc, const Frag& a, const Frag& b) {
#if defined(MS_ELEM_BF16)
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc, 0, 0, 0);
#elif defined(MS_ELEM_F16)
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a.v, b.v, acc, 0, 0, 0);
#else
#pragma unroll
    for (int i = 0; i < 8; ++i) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a.v[i], b.v[i], acc, 0, 0, 0);
#endif
}

// The value unchanged, but of unknown origin to the optimiser: a mask made this way is applied
// to a loaded value as it stands, where a visible condition would be turned into a branch round
// the load.
__device__ __forceinline__ int opaque(int x) {
    asm volatile("" : "+v"(x));
    return x;
}
__device__ __forceinline__ uint32_t opaque(uint32_t x) {
    asm volatile("" : "+v"(x));
    return x;
}

// A kernel's arguments are read through the scalar cache, which is empty when the kernel starts: every read is a
// trip to memory (about 0.4 us), and the compiler asks for an argument only where it is first needed, behind
// the branches and the waits that come before: one trip after the other (four in the fused decode attention).
// Naming the arguments here, first thing in a kernel, makes one request of them all.
template <typename T>
__device__ __forceinline__ void argument_now(T v) {
    asm volatile("" ::"s"(v));
}
template <typename... T>
__device__ __forceinline__ void arguments_now(T... v) {
    (argument_now(v), ...);
}

// ---- the activation of a gated feed-forward ----------------------------------------
// act(g) = g * sigmoid(u): u = g is SiLU; u = 2 sqrt(2 / pi) (g + 0.044715 g^3) is the tanh form of GELU,
// since 0.5 g (1 + tanh(z)) = g * sigmoid(2 z).  Which one is an argument of the products that apply it.
enum GateActivation { ACT_SILU = 0, ACT_GELU_TANH = 1, ACT_COUNT = 2 };
__device__ __forceinline__ float gate_activation(float g, int act) {
    const float u = act == ACT_GELU_TANH ? 1.5957691216057308f * (g + 0.044715f * g * g * g) : g;
#ifdef MS_ELEM_HALF
    // the hardware's reciprocal (one unit in the last place of 32 bits, far below the element type's rounding) for a
    // division, which is ten instructions an element in an epilogue that is all vector instructions
    return g * __builtin_amdgcn_rcpf(1.0f + __expf(-u));
#else
    return g / (1.0f + expf(-u));
#endif
}

// ---- reductions -----------------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
    return v;
}

// Sum over a block of NT threads (NT a multiple of 64, at most 1024); every thread gets
// the result.  `scratch` holds at least NT / 64 floats.  The order of the partial sums is
// fixed, so the result does not depend on timing.
template <int NT> __device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = wave_sum(v);
    const int w = threadIdx.x / WAVE;
    __syncthreads();
    if ((threadIdx.x & (WAVE - 1)) == 0) scratch[w] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < NT / WAVE; ++i) t += scratch[i];
    return t;
}

// ---- error channel --------------------------------------------------------------
// Entry points return 0 on success; otherwise ms_last_error() describes the refusal.
void set_error(const char* fmt, ...);
int check_launch(const char* what);
int compute_units();  // of the current device, asked once

#define MS_REQUIRE(cond, ...)            \
    do {                                 \
        if (!(cond)) {                   \
            ::ms::set_error(__VA_ARGS__); \
            return 1;                    \
        }                                \
    } while (0)

__host__ __device__ __forceinline__ int ceil_div(int a, int b) { return (a + b - 1) / b; }
__host__ __device__ __forceinline__ long ceil_div(long a, long b) { return (a + b - 1) / b; }

}  // namespace ms
