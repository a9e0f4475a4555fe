// Shared device/host helpers for the gfx950 TPA kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tpa_abi.h"

namespace tpa {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;
typedef __attribute__((ext_vector_type(8))) unsigned int u32x8;
typedef __attribute__((ext_vector_type(16))) unsigned int u32x16;
typedef __attribute__((ext_vector_type(8))) float f32x8;

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// bf16 bit pattern (in the low or high half of a dword) -> fp32
__device__ __forceinline__ float bf16lo_to_f32(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16hi_to_f32(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
__device__ __forceinline__ float bf16bits_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

// two fp32 -> packed bf16 pair (round to nearest even), lo in bits 0..15
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  bf16x2 r;
  r[0] = (__bf16)lo;
  r[1] = (__bf16)hi;
  return __builtin_bit_cast(uint32_t, r);
}

template <typename T>
__device__ __forceinline__ float load_as_f32(const T* p);
template <>
__device__ __forceinline__ float load_as_f32<float>(const float* p) {
  return *p;
}
template <>
__device__ __forceinline__ float load_as_f32<uint16_t>(const uint16_t* p) {
  return bf16bits_to_f32(*p);
}

template <typename T>
__device__ __forceinline__ void store_from_f32(T* p, float v);
template <>
__device__ __forceinline__ void store_from_f32<float>(float* p, float v) {
  *p = v;
}
template <>
__device__ __forceinline__ void store_from_f32<uint16_t>(uint16_t* p, float v) {
  __bf16 b = (__bf16)v;
  *p = __builtin_bit_cast(uint16_t, b);
}

// Combine a value with the one held by lane ^ 32.  v_permlane32_swap hands every lane both its
// own value and its partner's (which of the two results holds which depends on the half the
// lane is in), so order-independent reductions need no select.
__device__ __forceinline__ float halves_max(float x) {
  uint32_t u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float halves_sum(float x) {
  uint32_t u = __float_as_uint(x);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Minimum / maximum / sum of an int over the 64 lanes of a wave (every lane gets the result): what goes into a
// shared-memory atomic should be one value per wave - atomics of all lanes on one address are served one by one.
__device__ __forceinline__ int wave_min(int x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x = min(x, __shfl_xor(x, m, 64));
  return x;
}
__device__ __forceinline__ int wave_max(int x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x = max(x, __shfl_xor(x, m, 64));
  return x;
}
__device__ __forceinline__ int wave_sum(int x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x += __shfl_xor(x, m, 64);
  return x;
}

// Q fragments from rank factors: qf[ks] = bf16( scale * sum_r a[r] * b[r][16 ks + 0..7] ), where
// `ap` points at this lane's a[0] (rank stride a_stride) and `bp` at b[0][this lane's first
// element] (rank stride b_stride).  Ranks are taken G at a time with all 16-byte loads of the
// group in flight together, so the exposed memory latency is ceil(rq / G) round trips.
template <int NKS, int G>
__device__ __forceinline__ void build_q_fragments(const uint16_t* ap, int64_t a_stride, const uint16_t* bp, int64_t b_stride,
                                                  int rq, float scale, bf16x8 (&qf)[NKS]) {
  float acc[NKS][8];
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[ks][j] = 0.f;
  for (int r0 = 0; r0 < rq; r0 += G) {
    float a[G];
    u32x4 bv[G][NKS];
#pragma unroll
    for (int q = 0; q < G; ++q) {
      const int r = min(r0 + q, rq - 1);  // clamped reads past the last rank get weight 0
      a[q] = r0 + q < rq ? bf16bits_to_f32(ap[r * a_stride]) : 0.f;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) bv[q][ks] = *reinterpret_cast<const u32x4*>(bp + r * b_stride + 16 * ks);
    }
#pragma unroll
    for (int q = 0; q < G; ++q)
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[ks][2 * j] += a[q] * bf16lo_to_f32(bv[q][ks][j]);
          acc[ks][2 * j + 1] += a[q] * bf16hi_to_f32(bv[q][ks][j]);
        }
  }
#pragma unroll
  for (int ks = 0; ks < NKS; ++ks) {
    u32x4 packed;
#pragma unroll
    for (int j = 0; j < 4; ++j) packed[j] = pack_bf16(acc[ks][2 * j] * scale, acc[ks][2 * j + 1] * scale);
    qf[ks] = __builtin_bit_cast(bf16x8, packed);
  }
}

// Which of the eight (block, batch) pairs of round `round` the workgroups on XCD `xcd` take, with
// pair = block_rank * B + batch.  Workgroup ids map to XCDs statically, so with a fixed direction
// one XCD would collect the heaviest causal block of every round; odd rounds therefore reverse the
// order of the blocks.  Where B divides 8 only the block rank is reversed and the batch entry is
// kept, so that an XCD keeps meeting the same batch entries (their K/V factors stay in its L2);
// where B is a multiple of 8 a round holds one block rank only and nothing needs to move.
__device__ __forceinline__ int xcd_pair_slot(int round, int xcd, int B) {
  if (!(round & 1) || B % 8 == 0) return xcd;
  if (8 % B == 0) return (8 / B - 1 - xcd / B) * B + xcd % B;
  return 7 - xcd;
}

// Causal offset of a forward call as the kernels take it: row i sees keys <= i + offset.  Offsets
// of lk and more mask nothing and offsets of -lq and less mask everything, so the value is clamped
// to that range (keeps the kernels' index arithmetic far from overflow); 0 without the causal mask.
// With TPA_CAUSAL_BOTTOM_RIGHT the forward kernels add (keys of the batch entry - lq) themselves, since
// that differs per entry under kv_lengths; the range is then twice as wide.
inline int clamp_causal_offset(int offset, int lo, int hi) { return offset < lo ? lo : (offset > hi ? hi : offset); }
inline int causal_offset_of(const TpaFwdArgs* a) {
  if (!a->causal) return 0;
  if (a->causal == TPA_CAUSAL_BOTTOM_RIGHT) return clamp_causal_offset(a->causal_offset, -a->lq - a->lk, a->lq + a->lk);
  return clamp_causal_offset(a->causal_offset, -a->lq, a->lk);
}
// the backward takes no kv_lengths, so bottom-right alignment is the fixed offset lk - lq
inline int causal_offset_of(const TpaBwdArgs* a) {
  if (!a->causal) return 0;
  const int base = a->causal == TPA_CAUSAL_BOTTOM_RIGHT ? a->lk - a->lq : 0;
  return clamp_causal_offset(clamp_causal_offset(a->causal_offset, -a->lq - a->lk, a->lq + a->lk) + base, -a->lq, a->lk);
}

// Raise a kernel's dynamic LDS limit above the 64 KB a kernel gets without asking.  The attribute
// belongs to one device's copy of the code, so it is set once per device (`done` is the calling
// launcher's own table; a race between two first launches only repeats the same call).
constexpr int kMaxDevices = 64;
inline int raise_lds_limit(bool (&done)[kMaxDevices], const void* kern, size_t bytes) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) return TPA_ERR_LAUNCH;
  if (dev < kMaxDevices && done[dev]) return TPA_OK;
  if (hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) return TPA_ERR_LAUNCH;
  if (dev < kMaxDevices) done[dev] = true;
  return TPA_OK;
}

}  // namespace tpa

// host-side entry points of the individual kernel files (launchers return TPA_* codes)
int tpa_validate_fwd_args(const TpaFwdArgs* a);  // the checks every forward entry point makes first
int tpa_generic_launch(const TpaFwdArgs* a, hipStream_t stream);
int mha_generic_launch(const MhaFwdArgs* a, hipStream_t stream);
int tpa_prefill_mfma_supported(const TpaFwdArgs* a);
int tpa_prefill_mfma_launch(const TpaFwdArgs* a, hipStream_t stream);
int mha_prefill_mfma_supported(const MhaFwdArgs* a);
int mha_prefill_mfma_launch(const MhaFwdArgs* a, hipStream_t stream);
int tpa_prefill_f32_supported(const TpaFwdArgs* a);
int tpa_prefill_f32_launch(const TpaFwdArgs* a, hipStream_t stream);
int mha_prefill_f32_supported(const MhaFwdArgs* a);
int mha_prefill_f32_launch(const MhaFwdArgs* a, hipStream_t stream);
int tpa_nomat_pairs_supported(const TpaFwdArgs* a);
int tpa_nomat_pairs_launch(const TpaFwdArgs* a, hipStream_t stream);
int tpa_decode_mfma_supported(const TpaFwdArgs* a);
int tpa_decode_mfma_launch(const TpaFwdArgs* a, hipStream_t stream);
int tpa_decode_f32_supported(const TpaFwdArgs* a);
int tpa_decode_f32_launch(const TpaFwdArgs* a, hipStream_t stream);
// the same for a->lq query rows that are rows row0 .. row0 + a->lq - 1 of lq_total: a->qa / a->qb point at row row0,
// a->o / a->lse at row 0 of the full arrays, the causal mask counts rows from row0
int tpa_decode_mfma_launch_rows(const TpaFwdArgs* a, hipStream_t stream, int row0, int lq_total);
int tpa_decode_f32_launch_rows(const TpaFwdArgs* a, hipStream_t stream, int row0, int lq_total);
int mha_decode_supported(const MhaFwdArgs* a);
int mha_decode_launch(const MhaFwdArgs* a, hipStream_t stream);
int tpa_bwd_launch(const TpaBwdArgs* a, hipStream_t stream, int mfma);
int mha_bwd_launch(const MhaBwdArgs* a, hipStream_t stream, int mfma);
int dense_bwd_mfma_supported(int dtype, int dk, int dv, int64_t lq, int64_t lk, int64_t H, float sm_scale, const void* bias);
int dense_bwd_mfma_launch(const void* q, const void* k, const void* v, const void* d_o, const float* lse, const float* delta,
                          const int32_t* qseg, const int32_t* kvseg, float* dq, float* dk, float* dv, int B, int lq, int lk,
                          int H, int D, float sm_scale, int causal, int causal_offset, hipStream_t stream);
int dense_bwd_f32_supported(int dtype, int dk, int dv, int64_t lq, int64_t lk, const void* bias);
int dense_bwd_f32_launch(const float* q, const float* k, const float* v, const float* d_o, const float* lse, const float* delta,
                         const int32_t* qseg, const int32_t* kvseg, float* dq, float* dk, float* dv, int B, int lq, int lk,
                         int H, int D, float sm_scale, int causal, int causal_offset, hipStream_t stream);
size_t tpa_bwd_workspace_size(int64_t B, int64_t lq, int64_t lk, int64_t H, int64_t dk, int64_t dv);
size_t mha_bwd_workspace_size(int64_t B, int64_t lq, int64_t lk, int64_t H, int64_t dk, int64_t dv, int dtype);
size_t tpa_prefill_dense_bytes(int64_t B, int64_t lq, int64_t lk, int64_t H, int64_t D);
int tpa_prefill_wants_dense(int64_t lq, int64_t rk);
// dense bf16 X[B, L, H, D] = (scale/R) sum_r a_r (x) b_r from bf16 factors
int tpa_recon_dense_bf16(const TpaFactor* fa, const TpaFactor* fb, uint16_t* out, int B, int L, int H, int D, int R, float scale, hipStream_t stream);
// dense Q (times q_scale), K, V of a forward call in one launch; TPA_ERR_UNSUPPORTED where the vectorised kernel does not apply
int tpa_recon_dense_qkv_bf16(const TpaFwdArgs* a, uint16_t* qd, uint16_t* kd, uint16_t* vd, float q_scale, hipStream_t stream);
