// Instruction-level pieces shared by the eight-wave GEMM kernels (gemm_pair.hip, gemm_list.hip): explicit LDS
// fragment reads, direct-to-LDS loads, and matrix instructions on hand-numbered accumulation registers.
#pragma once
#include "common.h"

namespace mi {
namespace pair {

typedef __attribute__((address_space(3))) void *lptr_t;

template <int N>
__device__ __forceinline__ void wait_lgkm()
{
    asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory");
}
template <int N>
__device__ __forceinline__ void wait_vm()
{
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
template <int OFF>
__device__ __forceinline__ void ds_read128(v4i &dst, unsigned addr)
{
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(OFF));
}
// direct-to-LDS load of 16 bytes per lane: global address = sbase + voff, LDS address = ldsaddr + 16 * lane
__device__ __forceinline__ void dma16(const int8_t *sbase, unsigned voff, unsigned ldsaddr)
{
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(sbase), "s"(ldsaddr)
                 : "memory", "m0");
}
// accumulator (j, i) lives in a[4*(j*TM+i) .. +3]
template <int LO>
__device__ __forceinline__ void mfma_acc(const v4i &a, const v4i &b)
{
    asm volatile("v_mfma_i32_16x16x64_i8 a[%c2:%c3], %0, %1, a[%c2:%c3]" ::"v"(a), "v"(b), "n"(LO), "n"(LO + 3));
}
// the same with nothing to add to: the first instruction of a tile on its accumulator (no clearing pass, and no
// vector-ALU write in front of a matrix instruction that the hand-written code would have to pad)
template <int LO>
__device__ __forceinline__ void mfma_set(const v4i &a, const v4i &b)
{
    asm volatile("v_mfma_i32_16x16x64_i8 a[%c2:%c3], %0, %1, 0" ::"v"(a), "v"(b), "n"(LO), "n"(LO + 3));
}
template <int R>
__device__ __forceinline__ int acc_read()
{
    int v;
    asm volatile("v_accvgpr_read_b32 %0, a%c1" : "=v"(v) : "n"(R));
    return v;
}
template <int LO>
__device__ __forceinline__ v4i acc_read4()
{
    v4i v;
    v[0] = acc_read<LO>();
    v[1] = acc_read<LO + 1>();
    v[2] = acc_read<LO + 2>();
    v[3] = acc_read<LO + 3>();
    return v;
}
template <int R>
__device__ __forceinline__ void acc_zero()
{
    asm volatile("v_accvgpr_write_b32 a%c0, 0" ::"n"(R));
}

// ---- the same with the accumulators in ORDINARY registers v[ACC0 ..] that the compiler cannot allocate.
// The unified register file of this part lets a matrix instruction add into ordinary registers as well as into
// accumulation registers.  A kernel that carries __attribute__((amdgpu_num_vgpr(L / 2))), L <= ACC0, and uses no
// accumulation register is limited to v0 .. v(L-1) for everything the compiler places (a spill goes to scratch
// memory, which the build checks for), while v[ACC0 .. 255] are named by hand in the asm below and claimed for the
// wave by a clobber of v255 (the register count of the kernel's descriptor).  ACC0 = 128 leaves 128 accumulators (a wave
// tile of 4 x 8 matrix-instruction tiles) and 128 registers below them (fragments two K halves deep; the kernel may
// name some of the highest of these by hand as well and set its limit lower).  Unlike accumulation registers, which
// the register allocator may use to split a live range whenever ordinary registers run short, nothing but this
// code can write them.
namespace vacc {
constexpr int ACC0 = 128;
template <int LO>
__device__ __forceinline__ void mfma_acc(const v4i &a, const v4i &b)
{
    asm volatile("v_mfma_i32_16x16x64_i8 v[%c2:%c3], %0, %1, v[%c2:%c3]" ::"v"(a), "v"(b), "n"(ACC0 + LO), "n"(ACC0 + LO + 3));
}
// nothing to add to: the first instruction of a tile on its accumulator (no clearing pass)
template <int LO>
__device__ __forceinline__ void mfma_set(const v4i &a, const v4i &b)
{
    asm volatile("v_mfma_i32_16x16x64_i8 v[%c2:%c3], %0, %1, 0" ::"v"(a), "v"(b), "n"(ACC0 + LO), "n"(ACC0 + LO + 3));
}
template <int LO>
__device__ __forceinline__ void acc_zero4()
{
    asm volatile("v_mov_b32 v%c0, 0\n\tv_mov_b32 v%c1, 0\n\tv_mov_b32 v%c2, 0\n\tv_mov_b32 v%c3, 0" ::"n"(ACC0 + LO),
                 "n"(ACC0 + LO + 1), "n"(ACC0 + LO + 2), "n"(ACC0 + LO + 3));
}
// accumulator -> LDS, 16 bytes per lane, straight from its registers
template <int LO, int OFF>
__device__ __forceinline__ void acc_to_lds(unsigned addr)
{
    asm volatile("ds_write_b128 %0, v[%c1:%c2] offset:%3" ::"v"(addr), "n"(ACC0 + LO), "n"(ACC0 + LO + 3), "n"(OFF) : "memory");
}
// accumulator + o
template <int LO>
__device__ __forceinline__ v4i acc_plus(const v4i &o)
{
    v4i r;
    asm volatile("v_add_u32 %0, v%c2, %1" : "=v"(r[0]) : "v"(o[0]), "n"(ACC0 + LO));
    asm volatile("v_add_u32 %0, v%c2, %1" : "=v"(r[1]) : "v"(o[1]), "n"(ACC0 + LO + 1));
    asm volatile("v_add_u32 %0, v%c2, %1" : "=v"(r[2]) : "v"(o[2]), "n"(ACC0 + LO + 2));
    asm volatile("v_add_u32 %0, v%c2, %1" : "=v"(r[3]) : "v"(o[3]), "n"(ACC0 + LO + 3));
    return r;
}
}  // namespace vacc
__device__ __forceinline__ int ror8(int v) { return __builtin_amdgcn_update_dpp(v, v, 0x128, 0xf, 0xf, false); }

template <bool DEQ>
__device__ __forceinline__ void store4(float *y, int32_t *acc_out, int64_t idx, const v4i &v, float sxm, const float4 &s4)
{
    if constexpr (DEQ) {
        float4 o;
        o.x = ((float)v[0] * sxm) * s4.x;
        o.y = ((float)v[1] * sxm) * s4.y;
        o.z = ((float)v[2] * sxm) * s4.z;
        o.w = ((float)v[3] * sxm) * s4.w;
        *reinterpret_cast<float4 *>(y + idx) = o;
    } else {
        *reinterpret_cast<v4i *>(acc_out + idx) = v;
    }
}

}  // namespace pair
}  // namespace mi
