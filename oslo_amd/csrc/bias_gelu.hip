// Bias + GeLU (tanh form), forward and backward, for gfx950. The arithmetic is
// that of bias_gelu_fwb / bias_gelu_bwd (oslo/fused_kernels_utils.py:295-308)
// rewritten around the identity 0.5*(1 + tanh(u)) = 1/(1 + exp(-2u)), which
// needs one v_exp_f32 and one v_rcp_f32 per element. The backward also emits
// the bias gradient (a column sum), which the reference leaves to a separate
// full-tensor reduction by autograd (oslo/fused_kernels_utils.py:376-380).

#include <mutex>

#include "elementwise.hpp"
#include "gelu.hpp"

// Device memory of the entry point that takes no workspace argument
// (oslo_bias_gelu_bwd_static): the fp32 partial rows of the bias gradient live
// here instead of in a caller's buffer. Every GPU the library runs on holds its
// own copy of this array, at its own address, until the process ends. In host
// code the name is only a handle for hipGetSymbolAddress; kernels get the
// address that call returns.
static __device__ __align__(256) float scratch[OSLO_STATIC_WORKSPACE_BYTES / sizeof(float)];

namespace oslo {
namespace {

template <typename T, int VEC, int U, int OUT>
__global__ __launch_bounds__(kBlockThreads) void bias_gelu_fwd_kernel(
    T *out, const T *y, const T *__restrict__ bias, int64_t rows, int64_t cols,
    int col_tiles, int rows_per_block) {
  const EwPos pos = ew_position<VEC>(col_tiles, rows_per_block);
  if (pos.c0 >= cols) return; // no barrier in this kernel
  const BufRsrc yrs = ew_rsrc<T>(y, pos, rows_per_block, rows, cols);
  RawVec<T, VEC> raw[U];
#pragma unroll
  for (int u = 0; u < U; ++u)
    raw[u] = buffer_load_raw<T, VEC, true>(yrs, ew_offset<T>(pos, u, cols));
  float b[VEC];
  load_f32_cached<T, VEC>(b, bias + pos.c0);
  // rows past the end were read as zeros and their stores are dropped by the
  // same bound, so the body has no branch
  const BufRsrc ors = ew_rsrc<T>(out, pos, rows_per_block, rows, cols);
  float t[U][VEC];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    raw_to_f32<T, VEC>(t[u], raw[u]);
#pragma unroll
    for (int j = 0; j < VEC; ++j) t[u][j] = gelu_fwd(t[u][j] + b[j]);
    buffer_store_f32<T, VEC, OUT>(ors, ew_offset<T>(pos, u, cols), t[u]);
  }
}

template <typename T, int VEC, int U, bool WANT_DBIAS, int OUT>
__global__ __launch_bounds__(kBlockThreads) void bias_gelu_bwd_kernel(
    T *dy, float *__restrict__ partial, const T *g, const T *y,
    const T *__restrict__ bias, int64_t rows, int64_t cols, int col_tiles,
    int rows_per_block) {
  const EwPos pos = ew_position<VEC>(col_tiles, rows_per_block);
  const bool col_ok = pos.c0 < cols;
  float acc[VEC];
#pragma unroll
  for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
  if (col_ok) {
    const BufRsrc grs = ew_rsrc<T>(g, pos, rows_per_block, rows, cols);
    const BufRsrc yrs = ew_rsrc<T>(y, pos, rows_per_block, rows, cols);
    RawVec<T, VEC> graw[U], yraw[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      graw[u] = buffer_load_raw<T, VEC, true>(grs, ew_offset<T>(pos, u, cols));
      yraw[u] = buffer_load_raw<T, VEC, true>(yrs, ew_offset<T>(pos, u, cols));
    }
    float b[VEC];
    load_f32_cached<T, VEC>(b, bias + pos.c0);
    // rows past the end were read as zeros (g = 0 makes their products 0, so
    // they add nothing to dbias) and their stores are dropped by the bound
    const BufRsrc drs = ew_rsrc<T>(dy, pos, rows_per_block, rows, cols);
    float tg[U][VEC], ty_[U][VEC];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      raw_to_f32<T, VEC>(tg[u], graw[u]);
      raw_to_f32<T, VEC>(ty_[u], yraw[u]);
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        tg[u][j] = gelu_grad(ty_[u][j] + b[j]) * tg[u][j];
        if constexpr (WANT_DBIAS) acc[j] += tg[u][j];
      }
      buffer_store_f32<T, VEC, OUT>(drs, ew_offset<T>(pos, u, cols), tg[u]);
    }
  }
  if constexpr (WANT_DBIAS)
    write_colsum_partial<VEC>(acc, partial, cols, pos);
}

constexpr int kGeluBwdUnroll = 4;
static_assert(kGeluBwdUnroll >= kBwdMinUnroll, "workspace bound");

template <typename T, int VEC>
int launch_fwd(T *out, const T *y, const T *bias, int64_t rows, int64_t cols,
               hipStream_t stream) {
  const EwPlan p = plan_elementwise(rows, cols / VEC, kFwdMaxTx, kFwdUnroll);
  if (!p.ok) return fail(OSLO_E_UNSUPPORTED, "bias_gelu_fwd: tensor too large for one launch");
  if (keep_output_cached(rows * cols * (int64_t)sizeof(T)))
    bias_gelu_fwd_kernel<T, VEC, kFwdUnroll, kOutKeep><<<p.grid, p.block, 0, stream>>>(
        out, y, bias, rows, cols, p.col_tiles, p.rows_per_block);
  else
    bias_gelu_fwd_kernel<T, VEC, kFwdUnroll, kOutStream><<<p.grid, p.block, 0, stream>>>(
        out, y, bias, rows, cols, p.col_tiles, p.rows_per_block);
  return check_launch("bias_gelu_fwd");
}

template <typename T, int VEC>
int launch_bwd(T *dy, T *dbias, float *ws, const T *g, const T *y,
               const T *bias, int64_t rows, int64_t cols, hipStream_t stream) {
  const EwPlan p = plan_elementwise(rows, cols / VEC, kBwdMaxTx, kGeluBwdUnroll);
  if (!p.ok) return fail(OSLO_E_UNSUPPORTED, "bias_gelu_bwd: tensor too large for one launch");
  const bool keep = keep_output_cached(rows * cols * (int64_t)sizeof(T));
  auto go = [&]<bool WANT>() {
    if (keep)
      bias_gelu_bwd_kernel<T, VEC, kGeluBwdUnroll, WANT, kOutKeep>
          <<<p.grid, p.block, 0, stream>>>(dy, WANT ? ws : nullptr, g, y, bias, rows,
                                           cols, p.col_tiles, p.rows_per_block);
    else
      bias_gelu_bwd_kernel<T, VEC, kGeluBwdUnroll, WANT, kOutStream>
          <<<p.grid, p.block, 0, stream>>>(dy, WANT ? ws : nullptr, g, y, bias, rows,
                                           cols, p.col_tiles, p.rows_per_block);
  };
  if (dbias) {
    go.template operator()<true>();
    int s = check_launch("bias_gelu_bwd");
    if (s != OSLO_OK) return s;
    launch_colsum_finish<T>(dbias, ws, p.row_blocks, cols, stream);
    return check_launch("bias_gelu_bwd(dbias)");
  }
  go.template operator()<false>();
  return check_launch("bias_gelu_bwd");
}

// Address of `scratch` on the current device, looked up once per device.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float *g_scratch_ptr[kMaxDevices];

// `tensor`: one of the call's device tensors. Every GPU has a copy of the array
// at an address of its own, and the one looked up is the current device's: a
// call whose tensors live on another device is refused rather than handed a
// scratch address of the wrong GPU.
int static_scratch(float **out, const void *tensor) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return fail(OSLO_E_LAUNCH, "bias_gelu_bwd_static: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(OSLO_E_UNSUPPORTED, "bias_gelu_bwd_static: device %d, at most %d are tracked", dev, kMaxDevices);
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, tensor) == hipSuccess) {
    if (attr.type == hipMemoryTypeDevice && attr.device != dev)
      return fail(OSLO_E_BAD_ARG,
                  "bias_gelu_bwd_static: the tensors are on device %d, the current device is %d "
                  "(make the tensors' device current for the call)", attr.device, dev);
  } else {
    (void)hipGetLastError(); // a pointer the runtime does not know: the kernels will say
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    float *p = nullptr;
    e = hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return fail(OSLO_E_LAUNCH, "bias_gelu_bwd_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return OSLO_OK;
}

} // namespace
} // namespace oslo

extern "C" int oslo_bias_gelu_fwd(void *out, const void *y, const void *bias,
                                  int64_t rows, int64_t cols, int dtype,
                                  oslo_stream_t stream) {
  using namespace oslo;
  if (rows < 0 || cols < 0)
    return fail(OSLO_E_BAD_ARG, "bias_gelu_fwd: negative size");
  if (rows == 0 || cols == 0) return OSLO_OK;
  if (!out || !y || !bias)
    return fail(OSLO_E_BAD_ARG, "bias_gelu_fwd: null tensor");
  hipStream_t st = static_cast<hipStream_t>(stream);
  OSLO_DISPATCH_DTYPE(dtype, {
    constexpr int V = Io<T>::kVec;
    const bool vec = cols % V == 0 && aligned16(out) && aligned16(y) &&
                     aligned16(bias);
    T *o = static_cast<T *>(out);
    const T *yy = static_cast<const T *>(y);
    const T *bb = static_cast<const T *>(bias);
    return vec ? launch_fwd<T, V>(o, yy, bb, rows, cols, st)
               : launch_fwd<T, 1>(o, yy, bb, rows, cols, st);
  });
  return OSLO_OK;
}

extern "C" int oslo_bias_gelu_bwd(void *dy, void *dbias, float *workspace,
                                  const void *g, const void *y,
                                  const void *bias, int64_t rows, int64_t cols,
                                  int dtype, oslo_stream_t stream) {
  using namespace oslo;
  if (rows < 0 || cols < 0)
    return fail(OSLO_E_BAD_ARG, "bias_gelu_bwd: negative size");
  if (cols == 0) return OSLO_OK;
  if (dbias && !workspace && rows > 0)
    return fail(OSLO_E_BAD_ARG, "bias_gelu_bwd: dbias needs a workspace");
  if (rows > 0 && (!dy || !g || !y || !bias))
    return fail(OSLO_E_BAD_ARG, "bias_gelu_bwd: null tensor");
  hipStream_t st = static_cast<hipStream_t>(stream);
  OSLO_DISPATCH_DTYPE(dtype, {
    if (rows == 0) { // empty batch: the bias gradient is still defined (zero)
      if (dbias)
        launch_colsum_finish<T>(static_cast<T *>(dbias), nullptr, 0, cols, st); // writes zeros
      return check_launch("bias_gelu_bwd(dbias)");
    }
    constexpr int V = Io<T>::kVec;
    const bool vec = cols % V == 0 && aligned16(dy) && aligned16(g) &&
                     aligned16(y) && aligned16(bias) && aligned16(workspace);
    T *d = static_cast<T *>(dy);
    T *db = static_cast<T *>(dbias);
    const T *gg = static_cast<const T *>(g);
    const T *yy = static_cast<const T *>(y);
    const T *bb = static_cast<const T *>(bias);
    return vec ? launch_bwd<T, V>(d, db, workspace, gg, yy, bb, rows, cols, st)
               : launch_bwd<T, 1>(d, db, workspace, gg, yy, bb, rows, cols, st);
  });
  return OSLO_OK;
}

extern "C" int oslo_bias_gelu_bwd_static(void *dy, void *dbias, const void *g,
                                         const void *y, const void *bias,
                                         int64_t rows, int64_t cols, int dtype,
                                         oslo_stream_t stream) {
  using namespace oslo;
  if (rows < 0 || cols < 0)
    return fail(OSLO_E_BAD_ARG, "bias_gelu_bwd_static: negative size");
  const size_t need = dbias ? oslo_colsum_workspace_bytes(rows, cols) : 0;
  if (need > (size_t)OSLO_STATIC_WORKSPACE_BYTES)
    return fail(OSLO_E_UNSUPPORTED,
                "bias_gelu_bwd_static: [%lld, %lld] needs %zu bytes of workspace, the static "
                "buffer holds %zu; use oslo_bias_gelu_bwd with a workspace of the caller",
                (long long)rows, (long long)cols, need, (size_t)OSLO_STATIC_WORKSPACE_BYTES);
  float *ws = nullptr;
  if (dbias) {
    const int s = static_scratch(&ws, dy);
    if (s != OSLO_OK) return s;
  }
  // Every partial row the finishing sum reads is written by this call's first
  // kernel, so nothing in the buffer has to start at zero.
  return oslo_bias_gelu_bwd(dy, dbias, ws, g, y, bias, rows, cols, dtype, stream);
}
