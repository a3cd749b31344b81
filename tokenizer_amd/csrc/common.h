// Shared device helpers for the gfx950 kernels: storage types, wave reductions, launch checks.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define WAVE 64

// Storage element: float, or bfloat16 held as its 16 bits.  Arithmetic is always float.
struct bf16_t { uint16_t bits; };

__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits) { return __uint_as_float(bits << 16); }

// Round to nearest, ties to even; NaN stays NaN.
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float ld(const float* p) { return *p; }
__device__ __forceinline__ float ld(const bf16_t* p) { return bf16_bits_to_float(p->bits); }
__device__ __forceinline__ void st(float* p, float v) { *p = v; }
__device__ __forceinline__ void st(bf16_t* p, float v) { p->bits = float_to_bf16_bits(v); }

// The index of a thread's wave within its workgroup, as a scalar: conditions built from it are uniform
// branches.  Matrix instructions run whatever the lane mask says, so a matrix instruction must never sit
// in a block that the compiler enters by masking lanes; a condition that only looks divergent (one derived
// from threadIdx) can end up as exactly that.
__device__ __forceinline__ int wave_index() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

// HELD(a, b, ...): the listed kernel arguments are in scalar registers from this point on.  Left to itself the compiler
// fetches each piece of the argument block where it is first used, with a wait each time; a kernel that lists its
// arguments once, at its start, fetches them all in one trip.  (One statement for all of them: the fetches of a
// later statement would not be moved above an earlier one.)
#define HELD_1(a) "s"(a)
#define HELD_2(a, ...) "s"(a), HELD_1(__VA_ARGS__)
#define HELD_3(a, ...) "s"(a), HELD_2(__VA_ARGS__)
#define HELD_4(a, ...) "s"(a), HELD_3(__VA_ARGS__)
#define HELD_5(a, ...) "s"(a), HELD_4(__VA_ARGS__)
#define HELD_6(a, ...) "s"(a), HELD_5(__VA_ARGS__)
#define HELD_7(a, ...) "s"(a), HELD_6(__VA_ARGS__)
#define HELD_8(a, ...) "s"(a), HELD_7(__VA_ARGS__)
#define HELD_9(a, ...) "s"(a), HELD_8(__VA_ARGS__)
#define HELD_10(a, ...) "s"(a), HELD_9(__VA_ARGS__)
#define HELD_11(a, ...) "s"(a), HELD_10(__VA_ARGS__)
#define HELD_12(a, ...) "s"(a), HELD_11(__VA_ARGS__)
#define HELD_13(a, ...) "s"(a), HELD_12(__VA_ARGS__)
#define HELD_14(a, ...) "s"(a), HELD_13(__VA_ARGS__)
#define HELD_15(a, ...) "s"(a), HELD_14(__VA_ARGS__)
#define HELD_16(a, ...) "s"(a), HELD_15(__VA_ARGS__)
#define HELD_17(a, ...) "s"(a), HELD_16(__VA_ARGS__)
#define HELD_18(a, ...) "s"(a), HELD_17(__VA_ARGS__)
#define HELD_19(a, ...) "s"(a), HELD_18(__VA_ARGS__)
#define HELD_20(a, ...) "s"(a), HELD_19(__VA_ARGS__)
#define HELD_21(a, ...) "s"(a), HELD_20(__VA_ARGS__)
#define HELD_22(a, ...) "s"(a), HELD_21(__VA_ARGS__)
#define HELD_23(a, ...) "s"(a), HELD_22(__VA_ARGS__)
#define HELD_24(a, ...) "s"(a), HELD_23(__VA_ARGS__)
#define HELD_PICK(_1, _2, _3, _4, _5, _6, _7, _8, _9, _10, _11, _12, _13, _14, _15, _16, _17, _18, _19, _20, _21, _22, \
                  _23, _24, name, ...) name
#define HELD(...)                                                                                                       \
  asm volatile("" ::HELD_PICK(__VA_ARGS__, HELD_24, HELD_23, HELD_22, HELD_21, HELD_20, HELD_19, HELD_18, HELD_17,     \
                              HELD_16, HELD_15, HELD_14, HELD_13, HELD_12, HELD_11, HELD_10, HELD_9, HELD_8, HELD_7,   \
                              HELD_6, HELD_5, HELD_4, HELD_3, HELD_2, HELD_1)(__VA_ARGS__))

// A load of an int that is the same for the whole wave, through the scalar unit: for tables that no kernel in flight
// writes (positions, block tables, row lists).  The scalar unit has a counter of its own, so waiting for such a
// value does not wait for the vector loads that are under way; the compiler takes this path by itself only
// while it can prove that nothing in the kernel may have written the memory, which `HELD` above ends.
__device__ __forceinline__ int scalar_int(const int* p) {
  typedef const int __attribute__((address_space(4))) * constant_int;
  return *(constant_int)(p);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `scratch` holds 16 floats.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const int n_waves = (blockDim.x + WAVE - 1) / WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < n_waves; ++w) total += scratch[w];
  return total;
}

// Sixteen rows of a matrix as a 16x16x32 matrix instruction wants them (lane (col, g): row col), read line by line.
// The memory pipeline works a load off cache line by cache line, so a load that touches eight rows' whole lines of
// 128 bytes streams far more than one that touches sixteen rows' half lines.  The rows are therefore read by two
// loads, one for rows 0-7 (`lower`) and one for rows 8-15 (`upper`), in each of which lane (col, g) brings row
// col % 8's sixteen bytes number 2 g + col / 8 of the line; `lines_to_rows` puts them right by one exchange between
// lanes eight apart (a rotation within the row of sixteen lanes, no LDS): `first` = the sixteen bytes 2 g of row
// col's line, `second` = the sixteen bytes 2 g + 1.  The other operand takes the same bytes of its rows.
typedef uint32_t word4 __attribute__((ext_vector_type(4)));
typedef __bf16 line_bf16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ void lines_to_rows(const word4& lower, const word4& upper, bool low_lane, line_bf16x8& first,
                                              line_bf16x8& second) {
  word4 got;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int send = (int)(low_lane ? upper[i] : lower[i]);
    got[i] = (uint32_t)__builtin_amdgcn_update_dpp(send, send, 0x128, 0xF, 0xF, false);   // row_ror:8: from the lane eight away
  }
  word4 a, b;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = low_lane ? lower[i] : got[i];
    b[i] = low_lane ? got[i] : upper[i];
  }
  first = __builtin_bit_cast(line_bf16x8, a);
  second = __builtin_bit_cast(line_bf16x8, b);
}

// The compute units of the device, asked of the runtime once (the same on every device of a machine); launchers
// that weigh a launch's workgroups against the device use this, never a number of their own.
static inline int compute_units() {
  static int count = 0;
  if (count == 0) {
    int device = 0, value = 0;
    if (hipGetDevice(&device) == hipSuccess &&
        hipDeviceGetAttribute(&value, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess && value > 0)
      count = value;
    else
      count = 256;
  }
  return count;
}

// Every launcher returns 0, or the HIP error code of its launch.
#define LAUNCH_STATUS() ((int)hipGetLastError())

enum { DT_F32 = 0, DT_BF16 = 1 };
