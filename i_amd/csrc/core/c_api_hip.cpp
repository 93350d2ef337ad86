// extern "C" wrappers for the device-level entry points declared in i_hip.h.
#include "../../../include/i_hip.h"
#include "../runtime/kernel_launch.h"
#include "error.h"

namespace {
int finish(const ihip::Err& e) {
  if (e.empty()) return 0;
  icore::set_error(e);
  return -1;
}
bool dtype_ok(int d) { return d == I_DTYPE_F32 || d == I_DTYPE_BF16; }
}  // namespace

#pragma GCC visibility push(default)
extern "C" {

int i_hip_attention(const void* q, const void* k, const void* v, void* o, int in_dtype, int out_dtype, size_t bh,
                    size_t nq, size_t nk, size_t d, size_t dv, float scale, void* stream) {
  if (!dtype_ok(in_dtype) || !dtype_ok(out_dtype)) return finish("unknown dtype");
  return finish(ihip::launch_attention(q, k, v, o, (ihip::DType)in_dtype, (ihip::DType)out_dtype, bh, nq, nk, d, dv,
                                       nullptr, scale, (hipStream_t)stream));
}

int i_hip_attention_ex(const void* q, const void* k, const void* v, void* o, int in_dtype, int out_dtype, size_t bh,
                       size_t nq, size_t nk, size_t d, size_t dv, float scale, size_t query_tile, size_t key_tile,
                       int f32_scale, void* stream) {
  if (!dtype_ok(in_dtype) || !dtype_ok(out_dtype)) return finish("unknown dtype");
  return finish(ihip::launch_attention(q, k, v, o, (ihip::DType)in_dtype, (ihip::DType)out_dtype, bh, nq, nk, d, dv,
                                       nullptr, scale, (hipStream_t)stream,
                                       ihip::AttentionOptions{query_tile, key_tile, f32_scale != 0}));
}

int i_hip_gemm_nt_bf16(const void* a, const void* b, float* c, size_t bh, size_t m, size_t n, size_t k, void* stream) {
  return finish(ihip::launch_gemm_nt_bf16(a, b, c, bh, m, n, k, (hipStream_t)stream));
}

int i_hip_gemm_nt_bf16_ex(const void* a, const void* b, void* c, int out_dtype, size_t bh, size_t m, size_t n, size_t k,
                          size_t tile_m, size_t tile_n, void* stream) {
  if (!dtype_ok(out_dtype)) return finish("unknown dtype");
  return finish(ihip::launch_gemm_nt_bf16(a, b, c, bh, m, n, k, (hipStream_t)stream, tile_m, tile_n, nullptr,
                                          (ihip::DType)out_dtype));
}

int i_hip_gemm_nn_bf16(const void* a, const void* b, float* c, size_t bh, size_t m, size_t n, size_t k, void* stream) {
  return finish(ihip::launch_gemm_nn_bf16(a, b, c, bh, m, n, k, (hipStream_t)stream));
}

int i_hip_gemm_nt_f32(const float* a, const float* b, float* c, size_t bh, size_t m, size_t n, size_t k, void* stream) {
  return finish(ihip::launch_gemm_nt_f32(a, b, c, bh, m, n, k, (hipStream_t)stream));
}

int i_hip_row_softmax(const float* x, float* y, size_t rows, size_t cols, void* stream) {
  return finish(ihip::launch_row_softmax(x, y, rows, cols, (hipStream_t)stream));
}

int i_hip_convert(const void* src, void* dst, int from_dtype, int to_dtype, size_t n, void* stream) {
  if (!dtype_ok(from_dtype) || !dtype_ok(to_dtype)) return finish("unknown dtype");
  return finish(ihip::launch_convert(src, dst, (ihip::DType)from_dtype, (ihip::DType)to_dtype, n, (hipStream_t)stream));
}


}  // extern "C"
#pragma GCC visibility pop
