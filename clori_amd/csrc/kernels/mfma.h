// Small device helpers shared by the gfx950 attention kernels: MFMA operand types,
// 16-byte global loads, wave64 lane exchange and bf16 conversion.
#ifndef YVEX_ROCM_KERNELS_MFMA_H
#define YVEX_ROCM_KERNELS_MFMA_H

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define YVEX_LOG2E 1.4426950408889634f
#define YVEX_LN2 0.6931471805599453f

__device__ inline u32x4 load_b128(const void *p) { return *reinterpret_cast<const u32x4 *>(p); }
__device__ inline u32x2 load_b64(const void *p) { return *reinterpret_cast<const u32x2 *>(p); }
// The same for data that is read once and is far more than the caches hold (the pages of a
// batch of sessions): with the non-temporal hint random 4 KB blocks arrive at 6.2 TB/s on this
// part where plain loads reach 5.7.  Data that the caches can keep between launches (a history
// of a few MB, the latent pool of one MLA step) is slower that way.
__device__ inline u32x4 stream_b128(const void *p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(p));
}
__device__ inline u32x2 stream_b64(const void *p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(p));
}

__device__ inline bf16x8 as_bf16x8(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }
__device__ inline short4v as_short4(u32x2 v) { return __builtin_bit_cast(short4v, v); }

// S(16x16) += A(16x32) * B(32x16): lane l supplies A[l%16][8*(l/16)..+7] and
// B[8*(l/16)..+7][l%16]; the result lane l holds C[4*(l/16)+i][l%16], i = 0..3.
__device__ inline floatx4 mfma_16x16x32(bf16x8 a, bf16x8 b, floatx4 c)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// C(16x16) += A(16x16) * B(16x16): lane l supplies A[l%16][4*(l/16)..+3] and
// B[4*(l/16)..+3][l%16].
__device__ inline floatx4 mfma_16x16x16(short4v a, short4v b, floatx4 c)
{
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0);
}

// C(32x32) += A(32x16) * B(16x32): lane l supplies A[l%32][8*(l/32)..+7] and
// B[8*(l/32)..+7][l%32]; the result lane l holds C[8*(i/4) + 4*(l/32) + i%4][l%32].
__device__ inline floatx16 mfma_32x32x16(bf16x8 a, bf16x8 b, floatx16 c)
{
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

__device__ inline float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ inline float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

__device__ inline float xor_lanes(float v, int mask) { return __shfl_xor(v, mask, 64); }

// A value combined with the one the lane 16 (32) away holds, on the vector ALU:
// v_permlane16_swap / v_permlane32_swap of two copies leave the even rows (the lower half) in
// one register and the odd rows (the upper half) in the other, in every lane, so a commutative
// combination of the two is the answer in both partners.  __shfl_xor takes a trip through the
// LDS permute network instead, which sits in the dependent chain of every softmax step.
// (The two results go through scalars: a bit cast applied directly to a vector element reads
// element 0 whatever the index with this compiler.)
__device__ inline float max_xor16(float v)
{
    const uint32_t bits = __builtin_bit_cast(uint32_t, v);
    const u32x2 r = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
    const uint32_t even = r.x, odd = r.y;
    return fmaxf(__builtin_bit_cast(float, even), __builtin_bit_cast(float, odd));
}
__device__ inline float max_xor32(float v)
{
    const uint32_t bits = __builtin_bit_cast(uint32_t, v);
    const u32x2 r = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
    const uint32_t lower = r.x, upper = r.y;
    return fmaxf(__builtin_bit_cast(float, lower), __builtin_bit_cast(float, upper));
}
__device__ inline float sum_xor16(float v)
{
    const uint32_t bits = __builtin_bit_cast(uint32_t, v);
    const u32x2 r = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
    const uint32_t even = r.x, odd = r.y;
    return __builtin_bit_cast(float, even) + __builtin_bit_cast(float, odd);
}
__device__ inline float sum_xor32(float v)
{
    const uint32_t bits = __builtin_bit_cast(uint32_t, v);
    const u32x2 r = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
    const uint32_t lower = r.x, upper = r.y;
    return __builtin_bit_cast(float, lower) + __builtin_bit_cast(float, upper);
}

// Round-to-nearest-even narrowing with the quiet-NaN policy of the reference codec
// (src/gguf/quant_scalar.c:131-143).
__device__ inline uint16_t bf16_bits(float v)
{
    uint32_t u = __builtin_bit_cast(uint32_t, v);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

// Two floats -> packed bf16 pair with the hardware's round-to-nearest-even convert
// (v_cvt_pk_bf16_f32).
__device__ inline uint32_t pack_bf16x2(float lo, float hi)
{
    typedef float floatx2 __attribute__((ext_vector_type(2)));
    const floatx2 f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

// Packs the upper halves of two floats whose lower 16 bits are known to be zero (small
// integers): exact, one v_perm_b32.
__device__ inline uint32_t pack_bf16x2_exact(float lo, float hi)
{
    return __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, hi), __builtin_bit_cast(uint32_t, lo),
                                 0x07060302u);
}

__device__ inline float bf16_to_f32(uint16_t b)
{
    return __builtin_bit_cast(float, (uint32_t)b << 16);
}

// Sigmoid output gate (src/backend/cuda/transformer_kernels.cu:353-364, applied after
// attention at src/runtime/decoder.c:1266-1269): the published bf16 value times
// 1 / (1 + exp(-gate)) in F32, rounded to bf16 again.
__device__ inline float sigmoid(float x)
{
    return __builtin_amdgcn_rcpf(1.0f + fast_exp2(x * -1.4426950408889634f));
}

// Four published values (two packed words) times the gates of the same four dims.
__device__ inline u32x2 gate_four(u32x2 w, const uint16_t *gate)
{
    const u32x2 g = load_b64(gate);
    u32x2 r;
    r.x = pack_bf16x2(__builtin_bit_cast(float, w.x << 16) * sigmoid(__builtin_bit_cast(float, g.x << 16)),
                      __builtin_bit_cast(float, w.x & 0xffff0000u) *
                          sigmoid(__builtin_bit_cast(float, g.x & 0xffff0000u)));
    r.y = pack_bf16x2(__builtin_bit_cast(float, w.y << 16) * sigmoid(__builtin_bit_cast(float, g.y << 16)),
                      __builtin_bit_cast(float, w.y & 0xffff0000u) *
                          sigmoid(__builtin_bit_cast(float, g.y & 0xffff0000u)));
    return r;
}

// true when a packed pair holds an infinity or a NaN
__device__ inline bool pair_not_finite(uint32_t w)
{
    return (w & 0x7f80u) == 0x7f80u || (w & 0x7f800000u) == 0x7f800000u;
}

typedef int i32x4 __attribute__((ext_vector_type(4)));

// Raw buffer descriptor over [base, base + bytes): stride 0, untyped dword format; loads
// past the range return zero.  All four words are made wave-uniform.
__device__ inline i32x4 raw_buffer(const void *base, uint32_t bytes)
{
    const uint64_t address = (uint64_t)base;
    i32x4 rsrc;
    rsrc.x = __builtin_amdgcn_readfirstlane((int)(uint32_t)address);
    rsrc.y = __builtin_amdgcn_readfirstlane((int)((uint32_t)(address >> 32) & 0xffffu));
    rsrc.z = __builtin_amdgcn_readfirstlane((int)bytes);
    rsrc.w = 0x00027000;
    return rsrc;
}

// One buffer load of 16 bytes per lane that writes LDS directly: lane L's data lands at LDS
// byte address lds_address + 16 * L (M0 carries the wave-uniform destination).  Issued as
// opaque assembly on purpose: for the builtin form the compiler makes every later LDS read
// wait for all outstanding loads (it cannot see that ring buffers do not alias), which
// serialises any ring of tiles.  The caller waits with s_waitcnt vmcnt and a barrier.
__device__ inline void lds_dma_b128(uint32_t lds_address, i32x4 rsrc, uint32_t lane_offset,
                                    uint32_t uniform_offset)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %2, %1, %3 offen lds"
                 :
                 : "s"(lds_address), "s"(rsrc), "v"(lane_offset), "s"(uniform_offset)
                 : "memory");
}

// LDS byte address of a pointer into a __shared__ array.
__device__ inline uint32_t lds_address_of(const void *p)
{
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const unsigned char *)p;
}

#endif  // YVEX_ROCM_KERNELS_MFMA_H
