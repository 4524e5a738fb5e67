// Shared declarations for the gfx950 MLA / DSA kernels: vector types, error reporting, small
// device helpers.  Everything here is internal to the library; the exported C-ABI is declared in
// include/mla_hip.h.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mlahip {

// ---- error reporting -------------------------------------------------------------------------
// Entry points never throw: they return 0 or a negative code and leave a message that
// mlahip_last_error_string() hands back (thread-local).
enum : int {
  MLA_OK = 0,
  MLA_ERR_NULL = -1,      // a required pointer is null
  MLA_ERR_SHAPE = -2,     // a size / stride is out of the range the kernel supports
  MLA_ERR_UNSUPPORTED = -3,
  MLA_ERR_WORKSPACE = -4, // workspace too small
  MLA_ERR_LAUNCH = -100,  // the HIP runtime refused the launch
};
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);
// raises the dynamic-LDS limit of `kernel` to `bytes` on the current device (once per kernel and device)
int ensure_dynamic_lds(const void* kernel, int bytes, const char* what);

#define MLA_REQUIRE(cond, code, ...)                 \
  do {                                               \
    if (!(cond)) return ::mlahip::fail((code), __VA_ARGS__); \
  } while (0)

// ---- types -----------------------------------------------------------------------------------
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define LDS_PTR(T) __attribute__((address_space(3))) T*
#define GLB_PTR(T) __attribute__((address_space(1))) T*

constexpr int kPage = 128;    // tokens per cache page
constexpr int kDNope = 512;   // latent width (kv_lora_rank)
constexpr int kDRope = 64;    // rope width
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// ---- device helpers --------------------------------------------------------------------------
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// value held by lane (l ^ 32)
__device__ __forceinline__ float xor32(float v) { return __shfl_xor(v, 32, 64); }

// 16-byte global -> LDS copies that bypass the register file.  The LDS address is wave-uniform
// (it travels in M0): lane i's 16 bytes land at lds_addr + 16 * i.  They are written as inline
// assembly on purpose: the compiler then does not track them, so the only waits on them are the
// explicit MLA_WAIT_VMCNT() calls, which lets the copy of the next tile stay in flight while the
// current one is consumed.
__device__ __forceinline__ uint32_t lds_addr_of(const void* p) {
  return (uint32_t)(uintptr_t)(LDS_PTR(const char))(const char*)p;
}
// source = uniform 64-bit base + per-lane 32-bit byte offset
__device__ __forceinline__ void dma16_sv(const void* gbase_uniform, uint32_t voff, uint32_t lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_addr_uniform), "v"(voff), "s"(gbase_uniform)
               : "memory", "m0");
}
// the same with the LDS address given as a uniform base plus a compile-time constant (one scalar add straight into M0)
__device__ __forceinline__ void dma16_sv_m0add(const void* gbase_uniform, uint32_t voff, uint32_t lds_base_uniform, int lds_imm) {
  asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :
               : "s"(lds_base_uniform), "v"(voff), "s"(gbase_uniform), "n"(lds_imm)
               : "memory", "m0", "scc");
}
// The same two copies marked non-temporal, for bytes that are read once (the cache rows a decode launch streams): measured on
// the headline decode shape 1-2 us of 120 against the default policy; system scope (sc1, sc0 sc1) measured no different from
// the default.  Not for data that other workgroups on the XCD read at about the same time (queries, prefill tiles).
__device__ __forceinline__ void dma16_sv_nt(const void* gbase_uniform, uint32_t voff, uint32_t lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
               :
               : "s"(lds_addr_uniform), "v"(voff), "s"(gbase_uniform)
               : "memory", "m0");
}
__device__ __forceinline__ void dma16_sv_m0add_nt(const void* gbase_uniform, uint32_t voff, uint32_t lds_base_uniform, int lds_imm) {
  asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
               :
               : "s"(lds_base_uniform), "v"(voff), "s"(gbase_uniform), "n"(lds_imm)
               : "memory", "m0", "scc");
}
// source = per-lane 64-bit address
__device__ __forceinline__ void dma16_v(const void* gaddr, uint32_t lds_addr_uniform) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
               :
               : "s"(lds_addr_uniform), "v"(gaddr)
               : "memory", "m0");
}

// The same two copies issued by lanes 0..31 only (512 bytes): the upper half of the execution mask is cleared around
// the instruction inside the assembly, so the operands stay in the registers a uniform call site gives them.
__device__ __forceinline__ void dma16_sv_lo32(const void* gbase_uniform, uint32_t voff, uint32_t lds_addr_uniform) {
  uint32_t save;
  asm volatile("s_mov_b32 %0, exec_hi\n\ts_mov_b32 exec_hi, 0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3\n\ts_mov_b32 exec_hi, %0"
               : "=&s"(save)
               : "s"(lds_addr_uniform), "v"(voff), "s"(gbase_uniform)
               : "memory", "m0");
}
__device__ __forceinline__ void dma16_v_lo32(const void* gaddr, uint32_t lds_addr_uniform) {
  uint32_t save;
  asm volatile("s_mov_b32 %0, exec_hi\n\ts_mov_b32 exec_hi, 0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, off\n\ts_mov_b32 exec_hi, %0"
               : "=&s"(save)
               : "s"(lds_addr_uniform), "v"(gaddr)
               : "memory", "m0");
}

// One dword per lane by lanes 0..31 (128 bytes): lane i's dword lands at lds_addr + 4 * i.
__device__ __forceinline__ void dma4_sv_lo32(const void* gbase_uniform, uint32_t voff, uint32_t lds_addr_uniform) {
  uint32_t save;
  asm volatile("s_mov_b32 %0, exec_hi\n\ts_mov_b32 exec_hi, 0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %2, %3\n\ts_mov_b32 exec_hi, %0"
               : "=&s"(save)
               : "s"(lds_addr_uniform), "v"(voff), "s"(gbase_uniform)
               : "memory", "m0");
}

// Four dwords by lanes 0..3 (the rest of the execution mask is cleared around the instruction): lane i's dword lands at
// lds_addr + 4 * i.
__device__ __forceinline__ void dma4_sv_lanes4(const void* gbase_uniform, uint32_t voff, uint32_t lds_addr_uniform) {
  uint64_t save;
  asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, 15\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %2, %3\n\ts_mov_b64 exec, %0"
               : "=&s"(save)
               : "s"(lds_addr_uniform), "v"(voff), "s"(gbase_uniform)
               : "memory", "m0");
}
// the same by lanes 0..7
__device__ __forceinline__ void dma4_sv_lanes8(const void* gbase_uniform, uint32_t voff, uint32_t lds_addr_uniform) {
  uint64_t save;
  asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, 255\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %2, %3\n\ts_mov_b64 exec, %0"
               : "=&s"(save)
               : "s"(lds_addr_uniform), "v"(voff), "s"(gbase_uniform)
               : "memory", "m0");
}

// a 16-byte copy by lanes 0..7 only (128 bytes): lane i's bytes land at lds_addr + 16 * i
__device__ __forceinline__ void dma16_sv_lanes8(const void* gbase_uniform, uint32_t voff, uint32_t lds_addr_uniform) {
  uint64_t save;
  asm volatile("s_mov_b64 %0, exec\n\ts_mov_b64 exec, 255\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3\n\ts_mov_b64 exec, %0"
               : "=&s"(save)
               : "s"(lds_addr_uniform), "v"(voff), "s"(gbase_uniform)
               : "memory", "m0");
}

// Transposed LDS read: within each group of 16 lanes the 16 addresses name a 4 x 16 block of
// 16-bit elements (lane 4e+c points at row e, columns 4c..4c+3); lane j receives column j,
// i.e. the four rows' elements at that column.
__device__ __forceinline__ bf16x4 lds_read_tr16(const void* lds_addr) {
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 v4;
  v4 v = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((LDS_PTR(v4))lds_addr);
  return __builtin_bit_cast(bf16x4, v);
}

// Wait until at most n of this wave's global loads (LDS copies included) are outstanding.
#define MLA_WAIT_VMCNT(n) asm volatile("s_waitcnt vmcnt(" #n ")" ::: "memory")

// Workgroup barrier without the global-memory release fence of __syncthreads(): that fence waits for
// every outstanding global load, which would serialise the prefetch of the next K tile.  All data
// exchanged across the barrier lives in LDS; the caller waits for its own LDS copies (vmcnt) first.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

}  // namespace mlahip
