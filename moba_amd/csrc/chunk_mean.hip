// Key chunk-mean: kbar[f, h, :] = round( mean over the B tokens of filtered chunk f of K[., h, :] ),
// rounded once to the element type (bf16 or fp16).
//
// HBM-bound: K is read exactly once with 16-byte loads (a wave covers 1 KiB of
// one token row); the algorithmic traffic is S*H*D*2 bytes.  Accumulation is
// in fp64: the sum of a chunk of 16-bit float values is then exact, so the result
// does not depend on how the chunk is split over workgroups, and the rounded
// mean is reproducible bit for bit (fp64 -> fp32 -> element type, round to nearest even).
//
// Stage 1: grid (F, token splits, column blocks); each thread owns 8 adjacent
//          columns of the [H*D] token row and sums its share of a token split.
// Stage 2: sums the splits in order, divides by B, rounds.
#include <mutex>
#include "common.h"

namespace moba {

// cpb_log2: the workgroup's 256 threads are 1 << cpb_log2 column groups (8 adjacent columns each) times
// 256 >> cpb_log2 token lanes: a row narrower than 2048 elements still occupies every lane, and the token lanes'
// sums are added through LDS (exact sums: the order does not matter).
template <class E>
__global__ __launch_bounds__(256) void chunk_mean_partial_kernel(
    const typename E::elem* __restrict__ k, const int* __restrict__ fchunk_tok, double* __restrict__ partial,
    int HD8 /* H*D/8 */, int D8 /* D/8 */, int B, int nsplit, int tok_per_split, int64_t row_stride,
    int64_t head_stride, int batch_rows, int64_t batch_stride, int cpb_log2, int* __restrict__ clear,
    int64_t clear_ints) {
  MOBA_ELEM_TYPES(E)
  __shared__ double red[256 * 8];
  if (clear) {  // an int array of the caller's to be zeroed on the way (the workgroups share it out)
    const int64_t wg = blockIdx.x + (int64_t)gridDim.x * (blockIdx.y + (int64_t)gridDim.y * blockIdx.z);
    const int64_t step = (int64_t)gridDim.x * gridDim.y * gridDim.z * 256;
    for (int64_t i = wg * 256 + threadIdx.x; i < clear_ints; i += step) clear[i] = 0;
  }
  const int cpb = 1 << cpb_log2, lanes = 256 >> cpb_log2;
  const int tl = threadIdx.x >> cpb_log2;
  const int col = blockIdx.z * cpb + (threadIdx.x & (cpb - 1));
  const bool col_ok = col < HD8;
  const int split = blockIdx.y;
  const int f = blockIdx.x;  // the only grid dimension without a 65535 limit
  const int t0 = split * tok_per_split;
  const int t1 = min(B, t0 + tok_per_split);
  const int head = col_ok ? col / D8 : 0;
  // (a chunk lies inside one sequence, hence inside one batch entry of a batched layout)
  const int tok0 = fchunk_tok[f];
  const int be = batch_rows ? tok0 / batch_rows : 0;
  const elem* src = k + be * batch_stride + ((int64_t)(tok0 - be * batch_rows) + t0 + tl) * row_stride +
                    head * head_stride + (col_ok ? col - head * D8 : 0) * 8;
  const int64_t step = (int64_t)lanes * row_stride;
  double acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.0;
  int t = t0 + tl;
  if (col_ok) {
    for (; t + 7 * lanes < t1; t += 8 * lanes) {
      elem8 x[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) x[u] = __builtin_nontemporal_load(reinterpret_cast<const elem8*>(src + u * step));
      src += 8 * step;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        // sums of 16-bit float values are exact in fp64 whatever the order
        const double a = ((double)(float)x[0][e] + (double)(float)x[1][e]) + ((double)(float)x[2][e] + (double)(float)x[3][e]);
        const double b = ((double)(float)x[4][e] + (double)(float)x[5][e]) + ((double)(float)x[6][e] + (double)(float)x[7][e]);
        acc[e] += a + b;
      }
    }
    for (; t < t1; t += lanes) {
      elem8 x0 = *reinterpret_cast<const elem8*>(src);
      src += step;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += (double)(float)x0[e];
    }
  }
  if (lanes > 1) {  // (uniform)
#pragma unroll
    for (int e = 0; e < 8; ++e) red[e * 256 + threadIdx.x] = acc[e];
    __syncthreads();
    if (tl != 0) return;
    for (int l = 1; l < lanes; ++l)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += red[e * 256 + (l << cpb_log2) + threadIdx.x];
  }
  if (!col_ok) return;
  double* dst = partial + ((int64_t)(f * nsplit + split) * HD8 + col) * 8;
#pragma unroll
  for (int e = 0; e < 8; ++e) dst[e] = acc[e];
}

// fp64 -> fp32 rounded to odd (an inexact result gets the neighbour whose last bit is set): rounding that fp32
// value to bf16 or fp16 to nearest-even then gives what rounding the fp64 value once would, where two
// nearest-even roundings in a row can land on the wrong side of a tie.
__device__ __forceinline__ float round_to_odd_f32(double x) {
  float f = (float)x;  // nearest-even
  if ((double)f != x) {
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if (fabs((double)f) > fabs(x)) u -= 1;  // the neighbour toward zero (never crosses zero: |f| > |x| >= 0)
    u |= 1;
    f = __builtin_bit_cast(float, u);
  }
  return f;
}

template <class E>
__global__ __launch_bounds__(64) void chunk_mean_finish_kernel(
    const double* __restrict__ partial, typename E::elem* __restrict__ kbar, int HD8, int B, int nsplit, int F) {
  MOBA_ELEM_TYPES(E)
  // (one wave per workgroup: a small problem's few hundred outputs then spread over several compute units)
  const int64_t idx = (int64_t)blockIdx.x * 64 + threadIdx.x;  // over F * HD8
  if (idx >= (int64_t)F * HD8) return;
  const int f = (int)(idx / HD8);
  const int col = (int)(idx % HD8);
  double acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.0;
  const double* src = partial + ((int64_t)f * nsplit * HD8 + col) * 8;
  const int64_t step = (int64_t)HD8 * 8;
  int s = 0;
  for (; s + 4 <= nsplit; s += 4) {  // four splits' loads in flight together (nsplit is a power of two)
    double x[4][8];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int e = 0; e < 8; ++e) x[u][e] = src[u * step + e];
    src += 4 * step;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += (x[0][e] + x[1][e]) + (x[2][e] + x[3][e]);
  }
  for (; s < nsplit; ++s, src += step)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += src[e];
  elem8 o;
  const double inv = (double)B;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (elem)round_to_odd_f32(acc[e] / inv);
  *reinterpret_cast<elem8*>(kbar + idx * 8) = o;
}

}  // namespace moba

using namespace moba;

// column groups per workgroup (as a power of two): all 256 threads for rows of 2048 elements or more
static int pick_cpb_log2(int HD8) {
  int c = 0;
  while (c < 8 && (1 << c) < HD8) ++c;
  return c;
}
static int pick_nsplit(int HD8, int F, int B) {
  const int cpb_log2 = pick_cpb_log2(HD8);
  const int colblocks = (HD8 + (1 << cpb_log2) - 1) >> cpb_log2;
  const int lanes = 256 >> cpb_log2;
  int nsplit = 1;
  // enough workgroups to keep every CU's memory pipeline full (8 row loads in flight per lane),
  // few enough that the fp64 partial sums stay a small fraction of the traffic
  while ((int64_t)colblocks * F * nsplit < 1536 && B / (nsplit * 2) >= 64 && B / (nsplit * 2) >= 8 * lanes) nsplit *= 2;
  return nsplit;
}

extern "C" size_t moba_chunk_mean_workspace_bytes(int H, int D, int F, int B) {
  if (H <= 0 || D <= 0 || F <= 0 || B <= 0 || (H * D) % 8 != 0) return 0;
  const int HD8 = H * D / 8;
  return (size_t)F * pick_nsplit(HD8, F, B) * HD8 * 8 * sizeof(double);
}

static int launch_chunk_mean(const void* k, const int32_t* fchunk_tok, void* kbar, double* partial, int H, int D,
                             int F, int B, int nsplit, int64_t kts, int64_t khs, int batch_rows, int64_t kbs, int dtype,
                             int* clear, int64_t clear_ints, hipStream_t st) {
  LaunchCheck launch_check;
  const int HD8 = H * D / 8;
  const int tps = (B + nsplit - 1) / nsplit;
  const int cpb_log2 = pick_cpb_log2(HD8);
  dim3 grid(F, nsplit, (HD8 + (1 << cpb_log2) - 1) >> cpb_log2);
  const int64_t n = (int64_t)F * HD8;
  const dim3 fgrid((unsigned)((n + 63) / 64));
  if (dtype == MOBA_DTYPE_F16) {
    hipLaunchKernelGGL(chunk_mean_partial_kernel<F16>, grid, dim3(256), 0, st, (const f16*)k, fchunk_tok, partial,
                       HD8, D / 8, B, nsplit, tps, kts, khs, batch_rows, kbs, cpb_log2, clear, clear_ints);
    hipLaunchKernelGGL(chunk_mean_finish_kernel<F16>, fgrid, dim3(64), 0, st, (const double*)partial, (f16*)kbar,
                       HD8, B, nsplit, F);
  } else {
    hipLaunchKernelGGL(chunk_mean_partial_kernel<Bf16>, grid, dim3(256), 0, st, (const bf16*)k, fchunk_tok, partial,
                       HD8, D / 8, B, nsplit, tps, kts, khs, batch_rows, kbs, cpb_log2, clear, clear_ints);
    hipLaunchKernelGGL(chunk_mean_finish_kernel<Bf16>, fgrid, dim3(64), 0, st, (const double*)partial, (bf16*)kbar,
                       HD8, B, nsplit, F);
  }
  return launch_check.result();
}

// argument checks shared by the two entry points; kts, khs, kbr, kbs receive the key token and head strides, the
// rows per batch entry and the batch stride (elements)
static int check_chunk_mean_args(const void* k, const int32_t* fchunk_tok, void* kbar, int64_t S, int H, int D, int F,
                                 int B, const int64_t* strides, int dtype, int64_t& kts, int64_t& khs, int& kbr,
                                 int64_t& kbs) {
  if (dtype != MOBA_DTYPE_BF16 && dtype != MOBA_DTYPE_F16) return MOBA_ERR_UNSUPPORTED;
  if (!k || !fchunk_tok || !kbar || S <= 0 || H <= 0 || D <= 0 || F < 0 || B <= 0) return MOBA_ERR_ARG;
  if ((H * D) % 8 != 0 || ((uintptr_t)k & 15) || ((uintptr_t)kbar & 15)) return MOBA_ERR_ARG;
  if (D % 8 != 0) return MOBA_ERR_ARG;
  // strides (elements): {., ., k token, k head, rows per batch entry, ., k batch}; null = packed [S, H, D]
  kts = strides ? strides[2] : (int64_t)H * D;
  khs = strides ? strides[3] : D;
  if (strides && (strides[4] < 0 || strides[4] > 0x7fffffffLL)) return MOBA_ERR_ARG;  // (before it is narrowed)
  kbr = strides ? (int)strides[4] : 0;
  kbs = strides ? strides[6] : 0;
  if (kts <= 0 || khs <= 0 || (kts & 7) || (khs & 7)) return MOBA_ERR_ARG;
  if (kbr < 0 || (kbr > 0 && (kbs <= 0 || (kbs & 7)))) return MOBA_ERR_ARG;
  return MOBA_OK;
}

extern "C" int moba_chunk_mean(const void* k, const int32_t* fchunk_tok, void* kbar, void* workspace,
                               int64_t S, int H, int D, int F, int B, const int64_t* strides, int dtype,
                               int32_t* clear, int64_t clear_ints, void* stream) {
  if (clear_ints < 0 || (clear_ints > 0 && !clear)) return MOBA_ERR_ARG;
  if (F == 0) return MOBA_OK;  // (nothing to clear for: without chunks there are no lists to count)
  int64_t kts = 0, khs = 0, kbs = 0;
  int kbr = 0;
  const int rc = check_chunk_mean_args(k, fchunk_tok, kbar, S, H, D, F, B, strides, dtype, kts, khs, kbr, kbs);
  if (rc != MOBA_OK) return rc;
  if (!workspace || ((uintptr_t)workspace & 7)) return MOBA_ERR_ARG;
  return launch_chunk_mean(k, fchunk_tok, kbar, (double*)workspace, H, D, F, B, pick_nsplit(H * D / 8, F, B), kts, khs,
                           kbr, kbs, dtype, clear_ints > 0 ? clear : nullptr, clear_ints, (hipStream_t)stream);
}

// ---- the same stage for callers that cannot allocate: the partial sums live in a fixed array of the library ----
// Every GPU the library runs on holds its own copy of this array, at its own address, until the process
// ends.  The name below is a host-side stand-in, not a device address: host code only ever uses the
// address that hipGetSymbolAddress returned for the current device.
constexpr size_t kStaticPartialBytes = (size_t)32 << 20;
static __device__ __align__(256) double scratch[kStaticPartialBytes / sizeof(double)];

static std::mutex scratch_lock;
static double* scratch_of_device[kMaxDevices];   // guarded by scratch_lock

// device address of `scratch` on the current device (null on error), asked once per device
static double* static_partials() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0) return nullptr;
  std::lock_guard<std::mutex> hold(scratch_lock);
  if (dev < kMaxDevices && scratch_of_device[dev]) return scratch_of_device[dev];
  double* ptr = nullptr;
  if (hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) return nullptr;
  if (dev < kMaxDevices) scratch_of_device[dev] = ptr;
  return ptr;
}

extern "C" size_t moba_chunk_mean_static_capacity(void) { return kStaticPartialBytes; }

extern "C" int moba_chunk_mean_static(const void* k, const int32_t* fchunk_tok, void* kbar, int64_t S, int H, int D,
                                      int F, int B, const int64_t* strides, int dtype, void* stream) {
  if (F == 0) return MOBA_OK;
  int64_t kts = 0, khs = 0, kbs = 0;
  int kbr = 0;
  const int rc = check_chunk_mean_args(k, fchunk_tok, kbar, S, H, D, F, B, strides, dtype, kts, khs, kbr, kbs);
  if (rc != MOBA_OK) return rc;
  // The sums are exact in fp64, so the mean does not depend on the number of token splits: take the
  // widest split (up to the one moba_chunk_mean would use) whose partial sums fit the array.
  const int HD8 = H * D / 8;
  const size_t per_split = (size_t)F * HD8 * 8 * sizeof(double);
  if (per_split > kStaticPartialBytes) return MOBA_ERR_LIMIT;   // F * H * D * 8 bytes exceed the array
  int nsplit = pick_nsplit(HD8, F, B);
  while (nsplit > 1 && per_split * nsplit > kStaticPartialBytes) nsplit /= 2;
  double* partial = static_partials();
  if (!partial) return MOBA_ERR_LAUNCH;
  return launch_chunk_mean(k, fchunk_tok, kbar, partial, H, D, F, B, nsplit, kts, khs, kbr, kbs, dtype, nullptr, 0,
                           (hipStream_t)stream);
}
