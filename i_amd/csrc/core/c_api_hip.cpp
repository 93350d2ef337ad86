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
                                       nullptr, scale, (hipStream_t)stream, [&] {
                                         ihip::AttentionOptions options{query_tile, key_tile};
                                         options.knobs.attention_f32_scale = f32_scale != 0;
                                         return options;
                                       }()));
}

int i_hip_attention_opt(const void* q, const void* k, const void* v, void* o, int in_dtype, int out_dtype, size_t bh,
                        size_t nq, size_t nk, size_t d, size_t dv, float scale, size_t query_tile, size_t key_tile,
                        const char* options, void* stream) {
  if (!dtype_ok(in_dtype) || !dtype_ok(out_dtype)) return finish("unknown dtype");
  ihip::AttentionOptions opt{query_tile, key_tile};
  if (ihip::Err e = ihip::parse_kernel_options(options, &opt.knobs); !e.empty()) return finish(e);
  return finish(ihip::launch_attention(q, k, v, o, (ihip::DType)in_dtype, (ihip::DType)out_dtype, bh, nq, nk, d, dv,
                                       nullptr, scale, (hipStream_t)stream, opt));
}

int i_hip_gemm_opt(const void* a, const void* b, void* c, int in_dtype, int out_dtype, int b_row_major, size_t bh, size_t m,
                   size_t n, size_t k, const char* options, void* stream) {
  if (!dtype_ok(in_dtype) || !dtype_ok(out_dtype)) return finish("unknown dtype");
  ihip::KernelOptions knobs;
  if (ihip::Err e = ihip::parse_kernel_options(options, &knobs); !e.empty()) return finish(e);
  if (in_dtype == I_DTYPE_F32) {
    if (out_dtype != I_DTYPE_F32 || b_row_major) return finish("f32 products: row-major-transposed right operand and f32 output only");
    return finish(ihip::launch_gemm_nt_f32(static_cast<const float*>(a), static_cast<const float*>(b), static_cast<float*>(c), bh, m,
                                           n, k, (hipStream_t)stream, nullptr, nullptr, 1, knobs));
  }
  if (b_row_major)
    return finish(ihip::launch_gemm_nn_bf16(a, b, c, bh, m, n, k, (hipStream_t)stream, 0, 0, nullptr, (ihip::DType)out_dtype, nullptr,
                                            1, knobs));
  return finish(ihip::launch_gemm_nt_bf16(a, b, c, bh, m, n, k, (hipStream_t)stream, 0, 0, nullptr, (ihip::DType)out_dtype, knobs));
}

int i_hip_shader_clock_probe(void* ticks, unsigned microseconds, void* stream) {
  return finish(ihip::launch_shader_clock_probe(static_cast<unsigned long long*>(ticks), microseconds, (hipStream_t)stream));
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
