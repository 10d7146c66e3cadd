// Matrix-unit probe for gfx950: what v_mfma_f32_32x32x16_bf16 sustains on this GPU, alone and with ordinary vector
// instructions issued between the matrix instructions, from the same wave or from a second wave of the same SIMD.
// Measurement support for bench.py (libmvllm_probe.so, separate from the operator library): the prefill kernel is
// bound by the matrix unit, and its ceiling is what these loops reach at the clock the GPU sustains under this load,
// not the data-sheet product of units and boost clock.
//
// Every loop body is one asm block, so the instruction mix and order are exactly what is written here:
//   4 independent accumulator chains of MFMA (a chain's next instruction never waits for the one before it),
//   each MFMA followed by NV independent v_fma_f32 and NE v_exp_f32 on registers of their own.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __attribute__((ext_vector_type(16))) float v16f;
typedef __attribute__((ext_vector_type(8))) __bf16 v8bf16;

// One "slot": an MFMA on chain c, then the vector instructions of the mix.
#define FMA1(i) "v_fma_f32 %[x" #i "], %[x" #i "], %[k], %[x" #i "]\n\t"
#define EXP1(i) "v_exp_f32 %[x" #i "], %[x" #i "]\n\t"
#define MFMA(c, ab) "v_mfma_f32_32x32x16_bf16 %[c" #c "], %[a" #ab "], %[b" #ab "], %[c" #c "]\n\t"
#define V0
#define V2 FMA1(0) FMA1(1)
#define V3 FMA1(0) FMA1(1) FMA1(2)
#define V4 FMA1(0) FMA1(1) FMA1(2) FMA1(3)
#define V6 FMA1(0) FMA1(1) FMA1(2) FMA1(3) FMA1(4) FMA1(5)
#define V8 FMA1(0) FMA1(1) FMA1(2) FMA1(3) FMA1(4) FMA1(5) FMA1(6) FMA1(7)
#define E1 EXP1(8)
#define OPERANDS                                                                                                  \
  [c0] "+v"(c0), [c1] "+v"(c1), [c2] "+v"(c2), [c3] "+v"(c3), [x0] "+v"(x0), [x1] "+v"(x1), [x2] "+v"(x2),        \
      [x3] "+v"(x3), [x4] "+v"(x4), [x5] "+v"(x5), [x6] "+v"(x6), [x7] "+v"(x7), [x8] "+v"(x8)                    \
      : [a0] "v"(a0), [b0] "v"(b0), [a1] "v"(a1), [b1] "v"(b1), [k] "v"(k)
// the whole iteration is ONE asm statement: the compiler puts nothing between the instructions
#define MIXED(valu) asm volatile(MFMA(0, 0) valu MFMA(1, 1) valu MFMA(2, 0) valu MFMA(3, 1) valu : OPERANDS)
#define VECTOR_ONLY(valu) asm volatile(valu valu valu valu : OPERANDS)
// one accumulator chain (every MFMA waits for the one before it) and two chains
#define CHAIN1 asm volatile(MFMA(0, 0) MFMA(0, 1) MFMA(0, 0) MFMA(0, 1) : OPERANDS)
#define CHAIN2 asm volatile(MFMA(0, 0) MFMA(1, 1) MFMA(0, 0) MFMA(1, 1) : OPERANDS)

// MIX = 10 * (fmas per slot) + (exps per slot)
template <int MIX, bool DO_MFMA>
__device__ __forceinline__ void body(v16f& c0, v16f& c1, v16f& c2, v16f& c3, const v8bf16& a0, const v8bf16& b0,
                                     const v8bf16& a1, const v8bf16& b1, float& x0, float& x1, float& x2, float& x3,
                                     float& x4, float& x5, float& x6, float& x7, float& x8, float k) {
  if constexpr (DO_MFMA) {
    if constexpr (MIX == 0) MIXED(V0);
    if constexpr (MIX == 1001) CHAIN1;
    if constexpr (MIX == 1002) CHAIN2;
    if constexpr (MIX == 20) MIXED(V2);
    if constexpr (MIX == 30) MIXED(V3);
    if constexpr (MIX == 40) MIXED(V4);
    if constexpr (MIX == 60) MIXED(V6);
    if constexpr (MIX == 80) MIXED(V8);
    if constexpr (MIX == 1) MIXED(E1);
    if constexpr (MIX == 31) MIXED(V3 E1);
    if constexpr (MIX == 41) MIXED(V4 E1);
  } else {
    if constexpr (MIX == 20) VECTOR_ONLY(V2);
    if constexpr (MIX == 30) VECTOR_ONLY(V3);
    if constexpr (MIX == 40) VECTOR_ONLY(V4);
    if constexpr (MIX == 60) VECTOR_ONLY(V6);
    if constexpr (MIX == 80) VECTOR_ONLY(V8);
    if constexpr (MIX == 1) VECTOR_ONLY(E1);
    if constexpr (MIX == 31) VECTOR_ONLY(V3 E1);
    if constexpr (MIX == 41) VECTOR_ONLY(V4 E1);
  }
}

// ROLE 0: every wave runs the mixed body.  ROLE 1: two waves per SIMD, specialised: waves 0-3 of the workgroup run
// the MFMAs only, waves 4-7 (the second wave of each SIMD) the vector instructions only.  ROLE 2: every wave runs
// the vector instructions only (what they cost without the matrix unit).
template <int MIX, int ROLE>
__global__ __launch_bounds__(1024) void probe_kernel(float* out, int iters) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  v16f c0, c1, c2, c3;
  for (int i = 0; i < 16; ++i) c0[i] = c1[i] = c2[i] = c3[i] = 0.f;
  // operands: pseudo-random bf16 values in (-2, 2), two pairs used alternately, so that the multipliers see
  // changing inputs as they do in a real kernel (constant operands draw less power and flatter the clock)
  v8bf16 a0, b0, a1, b1;
  uint32_t h = (uint32_t)(blockIdx.x * 1024 + threadIdx.x) * 2654435761u + 12345u;
  auto next = [&]() {
    h ^= h << 13; h ^= h >> 17; h ^= h << 5;
    return (__bf16)(((float)(h & 0xffff) - 32768.f) * (1.f / 16384.f));
  };
  for (int i = 0; i < 8; ++i) { a0[i] = next(); b0[i] = next(); a1[i] = next(); b1[i] = next(); }
  float x0 = lane * 1e-3f, x1 = x0 + 1.f, x2 = x0 + 2.f, x3 = x0 + 3.f, x4 = x0 + 4.f, x5 = x0 + 5.f, x6 = x0 + 6.f,
        x7 = x0 + 7.f, x8 = -x0;
  const float k = 0.25f;
  const unsigned long long t0 = __builtin_amdgcn_s_memtime(), w0 = wall_clock64();
#define ARGS c0, c1, c2, c3, a0, b0, a1, b1, x0, x1, x2, x3, x4, x5, x6, x7, x8, k
  if (ROLE == 0) {
    for (int it = 0; it < iters; ++it) body<MIX, true>(ARGS);
  } else if (ROLE == 2) {
    for (int it = 0; it < iters; ++it) body<MIX, false>(ARGS);
  } else if (wave < 4) {
    for (int it = 0; it < iters; ++it) body<0, true>(ARGS);
  } else {
    for (int it = 0; it < iters; ++it) body<MIX, false>(ARGS);
  }
#undef ARGS
  const unsigned long long t1 = __builtin_amdgcn_s_memtime(), w1 = wall_clock64();
  if (blockIdx.x == 0 && threadIdx.x == 0) {      // shader clocks and 100 MHz ticks this wave spent in its loop
    out[1] = (float)(t1 - t0);
    out[2] = (float)(w1 - w0);
  }
  float s = x0 + x1 + x2 + x3 + x4 + x5 + x6 + x7 + x8;
  for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
  if (s == 12345.678f) out[0] = s;     // keeps the results alive; never true in practice
}

template <int MIX>
static int launch(int role, int waves_per_simd, int blocks, float* out, int iters, hipStream_t s) {
  const dim3 block(256 * waves_per_simd), grid(blocks);
  if (role == 0) probe_kernel<MIX, 0><<<grid, block, 0, s>>>(out, iters);
  else if (role == 1) probe_kernel<MIX, 1><<<grid, block, 0, s>>>(out, iters);
  else probe_kernel<MIX == 0 ? 40 : MIX, 2><<<grid, block, 0, s>>>(out, iters);
  return (int)hipGetLastError();
}

// One launch of `blocks` workgroups of 4 * waves_per_simd waves; every wave runs `iters` iterations of 4 slots, a slot
// being one MFMA + nv v_fma_f32 + ne v_exp_f32 (role 0), the two halves on different waves of a SIMD (role 1, needs
// waves_per_simd == 2), or the vector half alone (role 2).  (nv, ne) in {(0,0) (2,0) (3,0) (4,0) (6,0) (8,0) (0,1)
// (3,1) (4,1)}; (100,1) and (100,2): MFMAs only, on one and on two accumulator chains instead of four.  Returns 0, -1 for an unsupported mix, or a hipError_t.
extern "C" int mvllm_probe_mfma_mix(int nv, int ne, int role, int waves_per_simd, int blocks, float* out, int iters,
                                    void* stream) {
  hipStream_t s = (hipStream_t)stream;
  if (waves_per_simd < 1 || waves_per_simd > 4 || (role == 1 && waves_per_simd != 2) || role < 0 || role > 2 ||
      blocks <= 0 || iters <= 0 || !out)
    return -1;
  switch (10 * nv + ne) {
    case 0: return launch<0>(role, waves_per_simd, blocks, out, iters, s);
    case 20: return launch<20>(role, waves_per_simd, blocks, out, iters, s);
    case 30: return launch<30>(role, waves_per_simd, blocks, out, iters, s);
    case 40: return launch<40>(role, waves_per_simd, blocks, out, iters, s);
    case 60: return launch<60>(role, waves_per_simd, blocks, out, iters, s);
    case 80: return launch<80>(role, waves_per_simd, blocks, out, iters, s);
    case 1: return launch<1>(role, waves_per_simd, blocks, out, iters, s);
    case 31: return launch<31>(role, waves_per_simd, blocks, out, iters, s);
    case 41: return launch<41>(role, waves_per_simd, blocks, out, iters, s);
    case 1001: return launch<1001>(role, waves_per_simd, blocks, out, iters, s);   // nv = 100, ne = 1: one MFMA chain
    case 1002: return launch<1002>(role, waves_per_simd, blocks, out, iters, s);   // nv = 100, ne = 2: two chains
  }
  return -1;
}
