// One matrix instruction on caller-supplied register images: the tool that pins the
// operand layouts written down in mfma_common.h.  A single wavefront loads, for every
// lane, the A/B/C (and scale or sparse-index) registers from memory, issues exactly
// one MFMA/SMFMAC and writes the D registers back.
#include "internal.h"
#include "mfma_common.h"

namespace {

struct RawArgs {
  const uint32_t *a, *b, *c, *aux0, *aux1;
  uint32_t *d;
};

template <typename V, int N>
__device__ inline V regs(const uint32_t *base, int lane, int stride) {
  V v;
  uint32_t tmp[N];
#pragma unroll
  for (int i = 0; i < N; i++) tmp[i] = base[lane * stride + i];
  __builtin_memcpy(&v, tmp, sizeof(V));
  return v;
}

template <typename V, int N>
__device__ inline void store_regs(uint32_t *base, int lane, V v) {
  uint32_t tmp[N];
  __builtin_memcpy(tmp, &v, sizeof(V));
#pragma unroll
  for (int i = 0; i < N; i++) base[lane * 16 + i] = tmp[i];
}

template <int KIND, int SEL0, int SEL1>
__global__ void __launch_bounds__(64) raw_dense_kernel(RawArgs p) {
  const int l = threadIdx.x;
  if constexpr (KIND == MI355_MFMA_F16_16x16x32) {
    auto d = __builtin_amdgcn_mfma_f32_16x16x32_f16(regs<half8v, 4>(p.a, l, 8), regs<half8v, 4>(p.b, l, 8), regs<f32x4v, 4>(p.c, l, 16), 0, 0, 0);
    store_regs<f32x4v, 4>(p.d, l, d);
  } else if constexpr (KIND == MI355_MFMA_BF16_16x16x32) {
    auto d = __builtin_amdgcn_mfma_f32_16x16x32_bf16(regs<bf16x8v, 4>(p.a, l, 8), regs<bf16x8v, 4>(p.b, l, 8), regs<f32x4v, 4>(p.c, l, 16), 0, 0, 0);
    store_regs<f32x4v, 4>(p.d, l, d);
  } else if constexpr (KIND == MI355_MFMA_F16_32x32x16) {
    auto d = __builtin_amdgcn_mfma_f32_32x32x16_f16(regs<half8v, 4>(p.a, l, 8), regs<half8v, 4>(p.b, l, 8), regs<f32x16v, 16>(p.c, l, 16), 0, 0, 0);
    store_regs<f32x16v, 16>(p.d, l, d);
  } else if constexpr (KIND == MI355_MFMA_BF16_32x32x16) {
    auto d = __builtin_amdgcn_mfma_f32_32x32x16_bf16(regs<bf16x8v, 4>(p.a, l, 8), regs<bf16x8v, 4>(p.b, l, 8), regs<f32x16v, 16>(p.c, l, 16), 0, 0, 0);
    store_regs<f32x16v, 16>(p.d, l, d);
  } else if constexpr (KIND == MI355_MFMA_I8_16x16x64) {
    auto d = __builtin_amdgcn_mfma_i32_16x16x64_i8(regs<i32x4v, 4>(p.a, l, 8), regs<i32x4v, 4>(p.b, l, 8), regs<i32x4v, 4>(p.c, l, 16), 0, 0, 0);
    store_regs<i32x4v, 4>(p.d, l, d);
  } else {
    constexpr int FMT = KIND == MI355_MFMA_FP8_16x16x128 ? MI355_F8F6F4_E4M3
                      : KIND == MI355_MFMA_BF8_16x16x128 ? MI355_F8F6F4_E5M2
                      : KIND == MI355_MFMA_MXFP6_E2M3 ? MI355_F8F6F4_E2M3
                      : KIND == MI355_MFMA_MXFP6_E3M2 ? MI355_F8F6F4_E3M2 : MI355_F8F6F4_E2M1;
    auto d = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(regs<i32x8v, 8>(p.a, l, 8), regs<i32x8v, 8>(p.b, l, 8),
                                                              regs<f32x4v, 4>(p.c, l, 16), FMT, FMT, SEL0,
                                                              (int)p.aux0[l], SEL1, (int)p.aux1[l]);
    store_regs<f32x4v, 4>(p.d, l, d);
  }
}

// ABID = SEL0.  a: 4 dwords per lane, b: 8 dwords per lane, idx in aux0.
template <int KIND, int SEL0>
__global__ void __launch_bounds__(64) raw_sparse_kernel(RawArgs p) {
  const int l = threadIdx.x;
  const int idx = (int)p.aux0[l];
  if constexpr (KIND == MI355_SMFMAC_F16_16x16x64) {
    auto d = __builtin_amdgcn_smfmac_f32_16x16x64_f16(regs<half8v, 4>(p.a, l, 4), regs<half16v, 8>(p.b, l, 8), regs<f32x4v, 4>(p.c, l, 16), idx, 0, SEL0);
    store_regs<f32x4v, 4>(p.d, l, d);
  } else if constexpr (KIND == MI355_SMFMAC_BF16_16x16x64) {
    auto d = __builtin_amdgcn_smfmac_f32_16x16x64_bf16(regs<bf16x8v, 4>(p.a, l, 4), regs<bf16x16v, 8>(p.b, l, 8), regs<f32x4v, 4>(p.c, l, 16), idx, 0, SEL0);
    store_regs<f32x4v, 4>(p.d, l, d);
  } else if constexpr (KIND == MI355_SMFMAC_FP8_16x16x128) {
    auto d = __builtin_amdgcn_smfmac_f32_16x16x128_fp8_fp8(regs<i32x4v, 4>(p.a, l, 4), regs<i32x8v, 8>(p.b, l, 8), regs<f32x4v, 4>(p.c, l, 16), idx, 0, SEL0);
    store_regs<f32x4v, 4>(p.d, l, d);
  } else if constexpr (KIND == MI355_SMFMAC_BF8_16x16x128) {
    auto d = __builtin_amdgcn_smfmac_f32_16x16x128_bf8_bf8(regs<i32x4v, 4>(p.a, l, 4), regs<i32x8v, 8>(p.b, l, 8), regs<f32x4v, 4>(p.c, l, 16), idx, 0, SEL0);
    store_regs<f32x4v, 4>(p.d, l, d);
  } else {
    auto d = __builtin_amdgcn_smfmac_i32_16x16x128_i8(regs<i32x4v, 4>(p.a, l, 4), regs<i32x8v, 8>(p.b, l, 8), regs<i32x4v, 4>(p.c, l, 16), idx, 0, SEL0);
    store_regs<i32x4v, 4>(p.d, l, d);
  }
}

template <int KIND, int SEL0>
void dense_sel1(int sel1, RawArgs p, hipStream_t st) {
  switch (sel1) {
    case 0: raw_dense_kernel<KIND, SEL0, 0><<<1, 64, 0, st>>>(p); break;
    case 1: raw_dense_kernel<KIND, SEL0, 1><<<1, 64, 0, st>>>(p); break;
    case 2: raw_dense_kernel<KIND, SEL0, 2><<<1, 64, 0, st>>>(p); break;
    default: raw_dense_kernel<KIND, SEL0, 3><<<1, 64, 0, st>>>(p); break;
  }
}
template <int KIND>
void dense_sel(int sel0, int sel1, RawArgs p, hipStream_t st) {
  if constexpr (KIND < MI355_MFMA_FP8_16x16x128) {
    raw_dense_kernel<KIND, 0, 0><<<1, 64, 0, st>>>(p);
  } else {
    switch (sel0) {
      case 0: dense_sel1<KIND, 0>(sel1, p, st); break;
      case 1: dense_sel1<KIND, 1>(sel1, p, st); break;
      case 2: dense_sel1<KIND, 2>(sel1, p, st); break;
      default: dense_sel1<KIND, 3>(sel1, p, st); break;
    }
  }
}
template <int KIND>
void sparse_sel(int sel0, RawArgs p, hipStream_t st) {
  switch (sel0) {
    case 0: raw_sparse_kernel<KIND, 0><<<1, 64, 0, st>>>(p); break;
    case 1: raw_sparse_kernel<KIND, 1><<<1, 64, 0, st>>>(p); break;
    case 2: raw_sparse_kernel<KIND, 2><<<1, 64, 0, st>>>(p); break;
    default: raw_sparse_kernel<KIND, 3><<<1, 64, 0, st>>>(p); break;
  }
}

}  // namespace

extern "C" int mi355_mfma_raw(mi355_dev *dev, int sparse, int kind, const uint32_t *a_regs, const uint32_t *b_regs,
                              const uint32_t *c_regs, const uint32_t *aux0, const uint32_t *aux1, int sel0, int sel1,
                              uint32_t *d_regs) {
  MI355_ENTER(dev);
  MI355_REQUIRE(dev, a_regs && b_regs && c_regs && aux0 && aux1 && d_regs, "mfma_raw: null buffer");
  MI355_REQUIRE(dev, sel0 >= 0 && sel0 < 4 && sel1 >= 0 && sel1 < 4, "mfma_raw: selectors must be 0..3");
  RawArgs p{a_regs, b_regs, c_regs, aux0, aux1, d_regs};
  hipStream_t st = dev->stream;
  if (!sparse) {
    switch (kind) {
      case 0: dense_sel<0>(sel0, sel1, p, st); break;
      case 1: dense_sel<1>(sel0, sel1, p, st); break;
      case 2: dense_sel<2>(sel0, sel1, p, st); break;
      case 3: dense_sel<3>(sel0, sel1, p, st); break;
      case 4: dense_sel<4>(sel0, sel1, p, st); break;
      case 5: dense_sel<5>(sel0, sel1, p, st); break;
      case 6: dense_sel<6>(sel0, sel1, p, st); break;
      case 7: dense_sel<7>(sel0, sel1, p, st); break;
      case 8: dense_sel<8>(sel0, sel1, p, st); break;
      case 9: dense_sel<9>(sel0, sel1, p, st); break;
      default: return mi355_fail(dev, MI355_ERR_ARG, "mfma_raw: unknown dense kind %d", kind);
    }
  } else {
    switch (kind) {
      case 0: sparse_sel<0>(sel0, p, st); break;
      case 1: sparse_sel<1>(sel0, p, st); break;
      case 2: sparse_sel<2>(sel0, p, st); break;
      case 3: sparse_sel<3>(sel0, p, st); break;
      case 4: sparse_sel<4>(sel0, p, st); break;
      default: return mi355_fail(dev, MI355_ERR_ARG, "mfma_raw: unknown sparse kind %d", kind);
    }
  }
  MI355_LAUNCH_CHECK(dev, "mfma_raw");
  return MI355_OK;
}
