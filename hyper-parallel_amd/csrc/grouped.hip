// Device-side bookkeeping of the MoE grouped backward: everything that depends on the per-expert row counts is
// derived on the GPU from `offs`, so that no launch of the grouped path needs a host read of it.
//
// The weight gradient of expert e contracts over that expert's own tokens.  Its operands are the transposed
// 128x1 codes of grad_out and x, whose scaling groups run along the tokens and must restart at every expert's
// first row.  They are therefore laid out on a PADDED token axis: expert e owns max(1, ceil(rows_e / 128)) blocks
// of 128 tokens starting at a multiple of 128, the tail of its last block (an empty expert's whole block) holding
// zero codes, which add nothing to a sum.  The table below says where each expert's blocks lie; the grouped
// transposed quantizer and the grouped wgrad GEMM both read it.
#include "hpfp8_device.h"
#include "hpfp8_host.h"

namespace hpfp8 {

// layout (int32 words), E = experts, B = total_m / 128 + E padded blocks at most:
//   [4e + 0] first source row of expert e      [4e + 1] its row count (offsets clamped to [previous, total_m])
//   [4e + 2] its first padded block            [4e + 3] its number of padded blocks (>= 1)
//   [4E + i] the expert with the i-th largest block count (ties: lower index first): the order in which the
//            wgrad GEMM deals tiles to compute units, longest contractions first
//   [5E]     padded blocks in use
//   [5E + 1 + b] the expert that owns padded block b, -1 beyond the blocks in use
__global__ __launch_bounds__(1024) void grouped_layout_kernel(const int32_t* __restrict__ offs, int experts,
                                                              int total_m, int max_blocks, int32_t* __restrict__ layout) {
  // one workgroup; thread 0 walks the offsets (a prefix sum over at most 4096 experts), then everyone fills
  __shared__ int s_used;
  __shared__ int s_nb[4096], s_b0[4096];
  if (threadIdx.x == 0) {
    int prev = 0, blk = 0;
    for (int e = 0; e < experts; ++e) {
      int end = offs[e];
      end = end > prev ? end : prev;
      end = end < total_m ? end : total_m;
      const int rows = end - prev;
      const int nb = rows > 0 ? (rows + kBlock - 1) / kBlock : 1;
      layout[4 * e + 0] = prev;
      layout[4 * e + 1] = rows;
      layout[4 * e + 2] = blk;
      layout[4 * e + 3] = nb;
      s_nb[e] = nb;
      s_b0[e] = blk;
      blk += nb;
      prev = end;
    }
    layout[5 * experts] = blk;
    s_used = blk;
  }
  __syncthreads();
  const int used = s_used;
  for (int e = threadIdx.x; e < experts; e += blockDim.x) {
    const int nb = s_nb[e];
    int rank = 0;
    for (int j = 0; j < experts; ++j) {
      const int nj = s_nb[j];
      rank += (nj > nb || (nj == nb && j < e)) ? 1 : 0;
    }
    layout[4 * experts + rank] = e;
    const int b0 = s_b0[e];
    for (int b = 0; b < nb; ++b) layout[5 * experts + 1 + b0 + b] = e;
  }
  for (int b = used + threadIdx.x; b < max_blocks; b += blockDim.x) layout[5 * experts + 1 + b] = -1;
}

// rows [offs[experts - 1], total_m) of out[total_m, cols] (bf16, row stride ld elements) := 0: the rows of a grouped
// result that belong to no expert.  The workgroups share those rows out among themselves; with none, all leave at once.
__global__ __launch_bounds__(256) void zero_rows_after_kernel(uint16_t* __restrict__ out, const int32_t* __restrict__ offs,
                                                              int experts, int total_m, int cols, int64_t ld) {
  int last = 0;
  for (int e = 0; e < experts; ++e) {        // the clamped running maximum, as the GEMM reads the table
    const int v = offs[e];
    last = v > last ? v : last;
  }
  last = last < total_m ? last : total_m;
  const uint4 z = make_uint4(0, 0, 0, 0);
  for (int row = last + blockIdx.x; row < total_m; row += gridDim.x) {
    uint4* dst = reinterpret_cast<uint4*>(out + (int64_t)row * ld);
    for (int i = threadIdx.x; i < cols / 8; i += 256) dst[i] = z;
  }
}

}  // namespace hpfp8

using namespace hpfp8;

extern "C" {

int64_t hpfp8_grouped_layout_words(int experts, int64_t total_m) {
  if (experts < 0 || total_m < 0) return -1;
  return 5 * (int64_t)experts + 1 + (total_m / kBlock + experts);
}

int64_t hpfp8_grouped_padded_rows(int experts, int64_t total_m) {
  if (experts < 0 || total_m < 0) return -1;
  return (total_m / kBlock + experts) * kBlock;
}

int hpfp8_grouped_layout(const int32_t* offs, int experts, int64_t total_m, int32_t* layout, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(experts >= 0 && experts <= 4096, HPFP8_ERR_SHAPE, "grouped_layout: bad expert count %d", experts);
  HPFP8_REQUIRE(total_m >= 0 && total_m < (int64_t)0x7FFFFF00, HPFP8_ERR_SHAPE, "grouped_layout: bad row count");
  if (experts == 0) return HPFP8_OK;
  HPFP8_REQUIRE(offs && layout, HPFP8_ERR_ARG, "grouped_layout: null buffer");
  const int max_blocks = (int)(total_m / kBlock) + experts;
  grouped_layout_kernel<<<1, 1024, 0, (hipStream_t)stream>>>(offs, experts, (int)total_m, max_blocks, layout);
  return check_launch("grouped_layout");
}

int hpfp8_grouped_zero_unrouted_rows_bf16(void* out, int64_t ld, const int32_t* offs, int experts, int64_t total_m,
                                          int64_t cols, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(experts >= 0 && experts <= 4096, HPFP8_ERR_SHAPE, "grouped_zero_unrouted_rows: bad expert count %d", experts);
  HPFP8_REQUIRE(total_m >= 0 && total_m < (int64_t)0x7FFFFF00 && cols >= 0 && cols % 8 == 0 && ld >= cols && ld % 8 == 0,
                HPFP8_ERR_SHAPE, "grouped_zero_unrouted_rows: cols and ld must be multiples of 8, ld >= cols");
  const int64_t blocks = total_m < 1024 ? total_m : 1024;
  if (blocks == 0 || cols == 0) return HPFP8_OK;
  HPFP8_REQUIRE(out && (offs || experts == 0) && aligned16(out), HPFP8_ERR_ARG, "grouped_zero_unrouted_rows: null or misaligned buffer");
  zero_rows_after_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((uint16_t*)out, offs, experts, (int)total_m,
                                                                            (int)cols, ld);
  return check_launch("grouped_zero_unrouted_rows");
}

}  // extern "C"
