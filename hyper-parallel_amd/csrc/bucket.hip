// FP8 form of the flat gradient bucket, fused with its packing.
//
// The reference copies every parameter's gradient into one (shards x numel) buffer, row s holding
// chunk s of each gradient, casts that buffer to the reduce dtype, reduces it, casts the reduced row
// back, multiplies by grad_scale and copies the pieces out into the gradients again
// (hyper_parallel/core/hsdp/hsdp_grad_buffer.py:95-108 and :116-135).  Here the pack and the
// E4M3 quantization (1x128 groups along the row) are one pass over the gradients, and the
// dequantization and the unpack are one pass over the reduced row: the bf16 bucket is never
// materialised.
//
// Layout of a row: parameter e occupies elements [offset_e, offset_e + numel_e); offsets are
// multiples of 128 so a group never straddles two parameters; the gap up to the next offset is
// padding (zero codes; a padding-only group gets the scale of amax = 0).
#include "hpfp8_device.h"
#include "hpfp8_host.h"

namespace hpfp8 {

constexpr int kBucketBatch = 48;      // parameters per launch (the table travels as a kernel argument)
constexpr int kBucketUnroll = 4;      // 16-byte vectors per thread
constexpr int kBucketVecsPerWg = 256 * kBucketUnroll;

struct BucketBatch {
  const void* ptr[kBucketBatch];       // gradient of parameter e (pack: source, unpack: destination)
  int64_t numel[kBucketBatch];         // elements of one chunk of it (= elements it owns in a row)
  int64_t first_vec[kBucketBatch + 1]; // offset_e / 8; [count] = end of the span this launch covers
  int wg_first[kBucketBatch + 1];      // first workgroup (blockIdx.x) of parameter e
  int count;
};

// Workgroup -> (parameter, first vector inside that parameter's span).  Uniform scalar search.
__device__ __forceinline__ int bucket_locate(const BucketBatch& b, int wg, int64_t& vec0) {
  int e = 0;
  while (e + 1 < b.count && wg >= b.wg_first[e + 1]) ++e;
  vec0 = (int64_t)(wg - b.wg_first[e]) * kBucketVecsPerWg;
  return e;
}

__global__ __launch_bounds__(256) void bucket_pack_quant_kernel(const BucketBatch b, int64_t row_elems,
                                                                uint8_t* __restrict__ q,
                                                                float* __restrict__ scale,
                                                                float* __restrict__ scale_inv) {
  int64_t vec0;
  const int e = bucket_locate(b, blockIdx.x, vec0);
  const int shard = blockIdx.y;
  const int64_t n = b.numel[e];
  const int64_t span = b.first_vec[e + 1] - b.first_vec[e];       // vectors up to the next parameter
  const uint16_t* src = reinterpret_cast<const uint16_t*>(b.ptr[e]) + (int64_t)shard * n;
  const bool vec_ok = (reinterpret_cast<uintptr_t>(src) & 15) == 0;
  uint4 v[kBucketUnroll];
#pragma unroll
  for (int u = 0; u < kBucketUnroll; ++u) {
    const int64_t i = vec0 + u * 256 + threadIdx.x;   // vector inside the span
    const int64_t j = i * 8;                          // element inside the parameter's chunk
    v[u] = make_uint4(0, 0, 0, 0);
    if (i < span && j < n) {
      if (vec_ok && j + 8 <= n) {
        v[u] = nt_load16(src + j);
      } else {
        uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 8; ++t)
          if (j + t < n) w[t >> 1] |= (uint32_t)src[j + t] << (16 * (t & 1));
        v[u] = make_uint4(w[0], w[1], w[2], w[3]);
      }
    }
  }
  const int64_t row_vec0 = b.first_vec[e];
  static_assert(kBucketUnroll == 4, "scales4_from_amax serves four groups per 16-lane row");
  uint32_t m[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) m[u] = row16_max_u32(mag8(v[u]));
  const int l16 = threadIdx.x & 15;
  float s[4], mine, mine_inv;
  scales4_from_amax(m, l16, 0, s, mine, mine_inv);
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int64_t i = vec0 + u * 256 + threadIdx.x;
    if (i < span) nt_store8(q + (int64_t)shard * row_elems + (row_vec0 + i) * 8, cvt8<false>(v[u], s[u]));   // (row_vec0 + i: vector inside the row)
  }
  const int64_t i_mine = vec0 + l16 * 256 + threadIdx.x - l16;   // first vector of the group whose scales this lane holds
  if (l16 < 4 && i_mine < span) {
    const int64_t g = (int64_t)shard * (row_elems >> 7) + ((row_vec0 + i_mine) >> 4);
    if (scale) scale[g] = mine;
    scale_inv[g] = mine_inv;
  }
}

__global__ __launch_bounds__(256) void bucket_unpack_dequant_kernel(const BucketBatch b,
                                                                    const uint8_t* __restrict__ q,
                                                                    const float* __restrict__ scale_inv,
                                                                    float grad_scale, int apply_grad_scale) {
  int64_t vec0;
  const int e = bucket_locate(b, blockIdx.x, vec0);
  const int64_t n = b.numel[e];
  uint16_t* dst = reinterpret_cast<uint16_t*>(const_cast<void*>(b.ptr[e]));
  const bool vec_ok = (reinterpret_cast<uintptr_t>(dst) & 15) == 0;
  const int64_t row_vec0 = b.first_vec[e];
#pragma unroll
  for (int u = 0; u < kBucketUnroll; ++u) {
    const int64_t i = vec0 + u * 256 + threadIdx.x;
    const int64_t j = i * 8;
    if (j >= n) continue;                              // padding, or past this parameter
    const int64_t rv = row_vec0 + i;
    const u32x2 c = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(q + rv * 8));
    const float si = scale_inv[rv >> 4];
    const uint32_t words[2] = {c.x, c.y};
    uint32_t o[4];
#pragma unroll
    for (int wd = 0; wd < 2; ++wd) {
      v2f lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)words[wd], false);
      v2f hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)words[wd], true);
      float f[4] = {lo.x * si, lo.y * si, hi.x * si, hi.y * si};
      __bf16 h[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        h[t] = (__bf16)f[t];
        if (apply_grad_scale) h[t] = (__bf16)((float)h[t] * grad_scale);   // second rounding, as the reference's order
      }
      o[2 * wd] = (uint32_t)__builtin_bit_cast(uint16_t, h[0]) | ((uint32_t)__builtin_bit_cast(uint16_t, h[1]) << 16);
      o[2 * wd + 1] = (uint32_t)__builtin_bit_cast(uint16_t, h[2]) | ((uint32_t)__builtin_bit_cast(uint16_t, h[3]) << 16);
    }
    if (vec_ok && j + 8 <= n) {
      nt_store16(dst + j, make_uint4(o[0], o[1], o[2], o[3]));
    } else {
#pragma unroll
      for (int t = 0; t < 8; ++t)
        if (j + t < n) dst[j + t] = (uint16_t)(o[t >> 1] >> (16 * (t & 1)));
    }
  }
}

// Checks the table and launches `launch(batch, workgroups)` for runs of up to kBucketBatch parameters.
// cover_padding: workgroups also cover the gap after a parameter (pack writes zero codes there).
template <class F>
static int bucket_for_each_batch(const char* what, const void* const* ptrs, const int64_t* numels,
                                 const int64_t* offsets, int entries, int64_t row_elems, bool cover_padding, F launch) {
  HPFP8_REQUIRE(entries >= 0 && row_elems >= 0, HPFP8_ERR_SHAPE, "%s: negative size", what);
  HPFP8_REQUIRE(row_elems % kBlock == 0, HPFP8_ERR_SHAPE, "%s: row length %lld is not a multiple of 128", what,
                (long long)row_elems);
  if (entries == 0 || row_elems == 0) return HPFP8_OK;
  HPFP8_REQUIRE(ptrs && numels && offsets, HPFP8_ERR_ARG, "%s: null table", what);
  HPFP8_REQUIRE(offsets[0] == 0, HPFP8_ERR_SHAPE, "%s: the first offset must be 0", what);
  for (int e = 0; e < entries; ++e) {
    const int64_t next = e + 1 < entries ? offsets[e + 1] : row_elems;
    HPFP8_REQUIRE(offsets[e] % kBlock == 0, HPFP8_ERR_SHAPE, "%s: offset %lld of entry %d is not a multiple of 128", what,
                  (long long)offsets[e], e);
    HPFP8_REQUIRE(numels[e] > 0 && offsets[e] + numels[e] <= next, HPFP8_ERR_SHAPE,
                  "%s: entry %d (offset %lld, %lld elements) overlaps the next one or the end of the row", what, e,
                  (long long)offsets[e], (long long)numels[e]);
    HPFP8_REQUIRE(ptrs[e] != nullptr && (reinterpret_cast<uintptr_t>(ptrs[e]) & 1) == 0, HPFP8_ERR_ARG,
                  "%s: entry %d has a null or odd pointer", what, e);
  }
  for (int e0 = 0; e0 < entries; e0 += kBucketBatch) {
    BucketBatch b{};
    b.count = entries - e0 < kBucketBatch ? entries - e0 : kBucketBatch;
    int64_t wgs = 0;
    for (int i = 0; i < b.count; ++i) {
      const int e = e0 + i;
      const int64_t next = e + 1 < entries ? offsets[e + 1] : row_elems;
      b.ptr[i] = ptrs[e];
      b.numel[i] = numels[e];
      b.first_vec[i] = offsets[e] / 8;
      b.first_vec[i + 1] = next / 8;
      const int64_t vecs = cover_padding ? (next - offsets[e]) / 8 : (numels[e] + 7) / 8;
      b.wg_first[i] = (int)wgs;
      wgs += (vecs + kBucketVecsPerWg - 1) / kBucketVecsPerWg;
      HPFP8_REQUIRE(wgs < (int64_t)0x7FFFFFFF, HPFP8_ERR_SHAPE, "%s: bucket too large", what);
    }
    b.wg_first[b.count] = (int)wgs;
    int rc = launch(b, (unsigned)wgs);
    if (rc != HPFP8_OK) return rc;
  }
  return HPFP8_OK;
}

}  // namespace hpfp8

using namespace hpfp8;

extern "C" {

int hpfp8_bucket_pack_quantize_bf16(const void* const* grads, const int64_t* numels, const int64_t* offsets,
                                    int entries, int shards, int64_t row_elems, void* q, float* scale,
                                    float* scale_inv, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(shards >= 1 && shards <= 65535, HPFP8_ERR_SHAPE, "bucket_pack_quantize: shards must be in 1..65535");
  if (entries > 0 && row_elems > 0)
    HPFP8_REQUIRE(q && scale_inv && aligned16(q), HPFP8_ERR_ARG, "bucket_pack_quantize: null or misaligned output");
  return bucket_for_each_batch("bucket_pack_quantize", grads, numels, offsets, entries, row_elems, true,
                               [&](const BucketBatch& b, unsigned wgs) {
                                 bucket_pack_quant_kernel<<<dim3(wgs, (unsigned)shards), 256, 0, (hipStream_t)stream>>>(
                                     b, row_elems, (uint8_t*)q, scale, scale_inv);
                                 return check_launch("bucket_pack_quantize");
                               });
}

int hpfp8_bucket_unpack_dequantize_bf16(void* const* grads, const int64_t* numels, const int64_t* offsets,
                                        int entries, int64_t row_elems, const void* q, const float* scale_inv,
                                        float grad_scale, hpfp8_stream_t stream) {
  if (entries > 0 && row_elems > 0)
    HPFP8_REQUIRE(q && scale_inv && aligned16(q), HPFP8_ERR_ARG, "bucket_unpack_dequantize: null or misaligned input");
  return bucket_for_each_batch("bucket_unpack_dequantize", (const void* const*)grads, numels, offsets, entries,
                               row_elems, false, [&](const BucketBatch& b, unsigned wgs) {
                                 bucket_unpack_dequant_kernel<<<wgs, 256, 0, (hipStream_t)stream>>>(
                                     b, (const uint8_t*)q, scale_inv, grad_scale, grad_scale != 1.0f ? 1 : 0);
                                 return check_launch("bucket_unpack_dequantize");
                               });
}

}  // extern "C"
