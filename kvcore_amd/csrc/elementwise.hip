// Row-wise and element-wise kernels: embedding, RMSNorm with the residual sum,
// SiLU-mul, row gather, rotary tables, rotation fused with the paged K/V write,
// block-table updates.  All arithmetic is float32; storage is float32 or bfloat16.

#include <hip/hip_runtime.h>

#include <cstdio>
#include <mutex>
#include <string>

#include "device_utils.h"
#include "kvcore_hip.h"

using namespace kvc;

// ------------------------------------------------------------------ error plumbing
static thread_local std::string g_last_error;

int kvc_fail(const char* message) {
  g_last_error = message;
  return -1;
}

int kvc_check_launch(const char* what) {
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    g_last_error = std::string(what) + ": " + hipGetErrorString(err);
    return -2;
  }
  return 0;
}

int kvc_device_compute_units(void) {
  constexpr int kMaxDevices = 64;
  static int cached[kMaxDevices];  // 0: not asked yet
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return 256;
  if (cached[device] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || n <= 0) {
      (void)hipGetLastError();
      n = 256;
    }
    cached[device] = n;
  }
  return cached[device];
}

extern "C" int kvc_compute_units(void) { return kvc_device_compute_units(); }

extern "C" const char* kvc_last_error(void) { return g_last_error.c_str(); }
extern "C" int kvc_version(void) { return 1; }

static thread_local char g_variants[kVariantFamilies][64];

void kvc_note_variant(int family, const char* name) {
  if (family < 0 || family >= kVariantFamilies) return;
  snprintf(g_variants[family], sizeof(g_variants[family]), "%s", name);
}

extern "C" const char* kvc_last_variant(int family) {
  if (family < 0 || family >= kVariantFamilies) return "";
  return g_variants[family];
}

static inline hipStream_t S(kvc_stream s) { return reinterpret_cast<hipStream_t>(s); }

// ------------------------------------------------------------------------ embedding
template <typename T>
__global__ void embed_kernel(float* __restrict__ residual, const T* __restrict__ table,
                             const int32_t* __restrict__ ids, int H, int V, float scale) {
  const int t = blockIdx.x;
  const int id = ids[t];
  float* out = residual + static_cast<int64_t>(t) * H;
  if (id < 0 || id >= V) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = __uint_as_float(0x7fc00000u);
    return;
  }
  const T* row = table + static_cast<int64_t>(id) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = to_float(row[i]) * scale;
}

extern "C" int kvc_embed(float* residual, const void* table, const int32_t* ids, int T, int H,
                         int V, int dtype, float scale, kvc_stream stream) {
  if (T < 0 || H <= 0 || V <= 0) return kvc_fail("kvc_embed: bad sizes");
  if (T == 0) return 0;
  KVC_DISPATCH_DTYPE(dtype, Tp, hipLaunchKernelGGL(embed_kernel<Tp>, dim3(T), dim3(256), 0,
                                                   S(stream), residual,
                                                   static_cast<const Tp*>(table), ids, H, V, scale));
  return kvc_check_launch("kvc_embed");
}

// ------------------------------------------------------------- logits after the head
// x = logits + bias; x = cap * tanh(x / cap) when cap > 0; x *= scale.
template <typename TB>
__global__ void logits_finish_kernel(float* __restrict__ logits, int V, int64_t row_stride,
                                     const TB* __restrict__ bias, float soft_cap, float scale) {
  float* row = logits + static_cast<int64_t>(blockIdx.y) * row_stride;
  const int v = blockIdx.x * blockDim.x + threadIdx.x;
  if (v >= V) return;
  float x = row[v];
  if (bias != nullptr) x += to_float(bias[v]);
  if (soft_cap > 0.f) x = tanhf(x / soft_cap) * soft_cap;
  row[v] = x * scale;
}

extern "C" int kvc_logits_finish(float* logits, int S_, int V, int64_t row_stride, const void* bias,
                                 int bias_dtype, float soft_cap, float scale, kvc_stream stream) {
  if (S_ < 0 || V <= 0 || row_stride < V || S_ > 65535)
    return kvc_fail("kvc_logits_finish: bad sizes (at most 65535 rows)");
  if (soft_cap < 0.f) return kvc_fail("kvc_logits_finish: the soft cap must not be negative");
  if (S_ == 0) return 0;
  const dim3 grid((V + 255) / 256, S_);
  KVC_DISPATCH_DTYPE(bias_dtype, Tb,
                     hipLaunchKernelGGL(logits_finish_kernel<Tb>, grid, dim3(256), 0, S(stream), logits,
                                        V, row_stride, static_cast<const Tb*>(bias), soft_cap, scale));
  return kvc_check_launch("kvc_logits_finish");
}

// ------------------------------------------------------------------- filling of pages
// Every element of the listed pages, in all `outer` planes of a cache group's storage
// [outer, num_pages, page_elems], becomes the 16- or 32-bit pattern `bits`.
template <typename U>
__global__ void fill_pages_kernel(U* __restrict__ base, const int32_t* __restrict__ pages,
                                  int page_stride, int num_pages, int64_t page_elems, U bits) {
  const int page = pages[static_cast<int64_t>(blockIdx.x) * page_stride];
  if (page <= 0 || page >= num_pages) return;  // the null page is nobody's
  U* dst = base + (static_cast<int64_t>(blockIdx.y) * num_pages + page) * page_elems;
  for (int64_t i = threadIdx.x; i < page_elems; i += blockDim.x) dst[i] = bits;
}

extern "C" int kvc_fill_pages(void* storage, const int32_t* pages, int page_stride, int n, int outer,
                              int num_pages, int64_t page_elems, int elem_bytes, uint32_t bits,
                              kvc_stream stream) {
  if (n < 0 || page_stride <= 0 || outer <= 0 || outer > 65535 || num_pages <= 0 || page_elems <= 0)
    return kvc_fail("kvc_fill_pages: bad sizes");
  if (elem_bytes != 2 && elem_bytes != 4) return kvc_fail("kvc_fill_pages: elements of 2 or 4 bytes");
  if (n == 0) return 0;
  const dim3 grid(n, outer);
  if (elem_bytes == 2)
    hipLaunchKernelGGL(fill_pages_kernel<uint16_t>, grid, dim3(256), 0, S(stream),
                       static_cast<uint16_t*>(storage), pages, page_stride, num_pages, page_elems,
                       static_cast<uint16_t>(bits));
  else
    hipLaunchKernelGGL(fill_pages_kernel<uint32_t>, grid, dim3(256), 0, S(stream),
                       static_cast<uint32_t*>(storage), pages, page_stride, num_pages, page_elems, bits);
  return kvc_check_launch("kvc_fill_pages");
}

// -------------------------------------------------------------------------- RMSNorm
// One block per row.  Pass 1 forms the residual sum in float32, stores it and
// accumulates the squares; pass 2 reads the sums back (each thread its own) and scales.
template <typename T>
__global__ void add_rmsnorm_kernel(T* __restrict__ out, float* __restrict__ residual,
                                   const T* __restrict__ delta, const float* __restrict__ weight,
                                   float eps, int H) {
  __shared__ float scratch[16];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * H;
  float* r = residual + base;
  float ss = 0.f;
  if (delta != nullptr) {
    const T* dl = delta + base;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float v = r[i] + to_float(dl[i]);
      r[i] = v;
      ss += v * v;
    }
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float v = r[i];
      ss += v * v;
    }
  }
  const float total = block_sum(ss, scratch);
  const float inv = rsqrtf(total / static_cast<float>(H) + eps);
  T* o = out + base;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = from_float<T>(weight[i] * (r[i] * inv));
}

// Fast path for rows whose width is a multiple of 8: a thread keeps its 8-element chunks
// in registers, so residual and delta are read once, with 16- and 32-byte accesses that
// are all in flight together.  The order of the additions in the sum of squares is
// fixed by the width alone.
__device__ __forceinline__ void load8(const float* p, float* v) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  const float4 b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* p, float* v) {
  const uint4 a = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
__device__ __forceinline__ void store8(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void store8(bf16_t* p, const float* v) {
  uint4 a;
  a.x = f32_to_bf16_bits(v[0]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[1])) << 16);
  a.y = f32_to_bf16_bits(v[2]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[3])) << 16);
  a.z = f32_to_bf16_bits(v[4]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[5])) << 16);
  a.w = f32_to_bf16_bits(v[6]) | (static_cast<uint32_t>(f32_to_bf16_bits(v[7])) << 16);
  *reinterpret_cast<uint4*>(p) = a;
}

template <typename T, int NCH>
__global__ __launch_bounds__(256) void add_rmsnorm_vec_kernel(T* __restrict__ out,
                                                              float* __restrict__ residual,
                                                              const T* __restrict__ delta,
                                                              const float* __restrict__ weight,
                                                              float eps, int H) {
  __shared__ float scratch[16];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * H;
  float v[NCH][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e = (c * 256 + threadIdx.x) * 8;
    if (e < H) {
      load8(residual + base + e, v[c]);
      if (delta != nullptr) {
        float d[8];
        load8(delta + base + e, d);
#pragma unroll
        for (int i = 0; i < 8; ++i) v[c][i] += d[i];
        store8(residual + base + e, v[c]);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += v[c][i] * v[c][i];
    }
  }
  const float total = block_sum(ss, scratch);
  const float inv = rsqrtf(total / static_cast<float>(H) + eps);
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e = (c * 256 + threadIdx.x) * 8;
    if (e < H) {
      float w[8], y[8];
      load8(weight + e, w);
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] = w[i] * (v[c][i] * inv);
      store8(out + base + e, y);
    }
  }
}

template <typename T>
static bool launch_add_rmsnorm_vec(T* out, float* residual, const T* delta, const float* weight,
                                   float eps, int rows, int H, hipStream_t stream) {
  const auto misaligned = [](const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) != 0; };
  if (H % 8 || H > 8 * 2048 || misaligned(out, 16) || misaligned(residual, 16) ||
      misaligned(weight, 16) || (delta != nullptr && misaligned(delta, 16)))
    return false;
  const int nch = (H + 2047) / 2048;
#define KVC_NORM_CASE(NN)                                                                        \
  hipLaunchKernelGGL((add_rmsnorm_vec_kernel<T, NN>), dim3(rows), dim3(256), 0, stream, out,     \
                     residual, delta, weight, eps, H)
  if (nch <= 1) KVC_NORM_CASE(1);
  else if (nch <= 2) KVC_NORM_CASE(2);
  else if (nch <= 4) KVC_NORM_CASE(4);
  else KVC_NORM_CASE(8);
#undef KVC_NORM_CASE
  return true;
}

// The same with the pending output given as float32 partial sums [slices, rows, H] of a
// product cut along K (+ a bias): they are added up in slice order, then into the residual.
template <typename T, int NCH>
__global__ __launch_bounds__(256) void add_slices_rmsnorm_vec_kernel(
    T* __restrict__ out, float* __restrict__ residual, const float* __restrict__ partial, int slices,
    int64_t slice_stride, const bf16_t* __restrict__ bias, const float* __restrict__ weight, float eps,
    int H) {
  __shared__ float scratch[16];
  const int64_t base = static_cast<int64_t>(blockIdx.x) * H;
  float v[NCH][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e = (c * 256 + threadIdx.x) * 8;
    if (e < H) {
      float d[8];
      load8(partial + base + e, d);
      for (int s = 1; s < slices; ++s) {
        float p[8];
        load8(partial + s * slice_stride + base + e, p);
#pragma unroll
        for (int i = 0; i < 8; ++i) d[i] += p[i];
      }
      if (bias != nullptr) {
        float b[8];
        load8(bias + e, b);
#pragma unroll
        for (int i = 0; i < 8; ++i) d[i] += b[i];
      }
      load8(residual + base + e, v[c]);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[c][i] += d[i];
      store8(residual + base + e, v[c]);
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += v[c][i] * v[c][i];
    }
  }
  const float total = block_sum(ss, scratch);
  const float inv = rsqrtf(total / static_cast<float>(H) + eps);
#pragma unroll
  for (int c = 0; c < NCH; ++c) {
    const int e = (c * 256 + threadIdx.x) * 8;
    if (e < H) {
      float w[8], y[8];
      load8(weight + e, w);
#pragma unroll
      for (int i = 0; i < 8; ++i) y[i] = w[i] * (v[c][i] * inv);
      store8(out + base + e, y);
    }
  }
}

extern "C" int kvc_add_slices_rmsnorm(void* out, float* residual, const float* partial, int slices,
                                      const void* bias, const float* weight, float eps, int T, int H,
                                      int dtype, kvc_stream stream) {
  if (T < 0 || H <= 0 || slices < 1) return kvc_fail("kvc_add_slices_rmsnorm: bad sizes");
  const auto misaligned = [](const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) != 0; };
  if (H % 8 || H > 8 * 2048 || misaligned(out, 16) || misaligned(residual, 16) || misaligned(partial, 16) ||
      misaligned(weight, 16) || (bias != nullptr && misaligned(bias, 16)))
    return kvc_fail("kvc_add_slices_rmsnorm: the width must be a multiple of 8, at most 16384, and "
                    "the operands 16-byte aligned");
  if (dtype != 0 && dtype != 1) return kvc_fail("kvc_add_slices_rmsnorm: unknown dtype code");
  if (T == 0) return 0;
  const int nch = (H + 2047) / 2048;
  const int64_t stride = static_cast<int64_t>(T) * H;
  const bf16_t* b = static_cast<const bf16_t*>(bias);
#define KVC_NORM_CASE(TT, NN)                                                                       \
  hipLaunchKernelGGL((add_slices_rmsnorm_vec_kernel<TT, NN>), dim3(T), dim3(256), 0, S(stream),     \
                     static_cast<TT*>(out), residual, partial, slices, stride, b, weight, eps, H)
#define KVC_NORM_NCH(TT)                \
  if (nch <= 1) KVC_NORM_CASE(TT, 1);   \
  else if (nch <= 2) KVC_NORM_CASE(TT, 2); \
  else if (nch <= 4) KVC_NORM_CASE(TT, 4); \
  else KVC_NORM_CASE(TT, 8)
  if (dtype == 0) { KVC_NORM_NCH(float); } else { KVC_NORM_NCH(bf16_t); }
#undef KVC_NORM_NCH
#undef KVC_NORM_CASE
  return kvc_check_launch("kvc_add_slices_rmsnorm");
}

extern "C" int kvc_add_rmsnorm(void* out, float* residual, const void* delta, const float* weight,
                               float eps, int T, int H, int dtype, kvc_stream stream) {
  if (T < 0 || H <= 0) return kvc_fail("kvc_add_rmsnorm: bad sizes");
  if (T == 0) return 0;
  {
    bool done = false;
    if (dtype == 0)
      done = launch_add_rmsnorm_vec(static_cast<float*>(out), residual,
                                    static_cast<const float*>(delta), weight, eps, T, H, S(stream));
    else if (dtype == 1)
      done = launch_add_rmsnorm_vec(static_cast<bf16_t*>(out), residual,
                                    static_cast<const bf16_t*>(delta), weight, eps, T, H, S(stream));
    if (done) return kvc_check_launch("kvc_add_rmsnorm");
  }
  KVC_DISPATCH_DTYPE(dtype, Tp,
                     hipLaunchKernelGGL(add_rmsnorm_kernel<Tp>, dim3(T), dim3(256), 0, S(stream),
                                        static_cast<Tp*>(out), residual,
                                        static_cast<const Tp*>(delta), weight, eps, H));
  return kvc_check_launch("kvc_add_rmsnorm");
}

template <typename T>
__global__ void rmsnorm_kernel(T* __restrict__ out, const T* __restrict__ x,
                               const float* __restrict__ weight, float eps, int H,
                               int64_t x_stride, int64_t out_stride) {
  __shared__ float scratch[16];
  const T* xr = x + static_cast<int64_t>(blockIdx.x) * x_stride;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = to_float(xr[i]);
    ss += v * v;
  }
  const float total = block_sum(ss, scratch);
  const float inv = rsqrtf(total / static_cast<float>(H) + eps);
  T* o = out + static_cast<int64_t>(blockIdx.x) * out_stride;
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    o[i] = from_float<T>(weight[i] * (to_float(xr[i]) * inv));
}

extern "C" int kvc_rmsnorm(void* out, const void* x, const float* weight, float eps, int T, int H,
                           int64_t x_stride, int64_t out_stride, int dtype, kvc_stream stream) {
  if (T < 0 || H <= 0 || x_stride < H || out_stride < H) return kvc_fail("kvc_rmsnorm: bad sizes");
  if (T == 0) return 0;
  KVC_DISPATCH_DTYPE(dtype, Tp,
                     hipLaunchKernelGGL(rmsnorm_kernel<Tp>, dim3(T), dim3(256), 0, S(stream),
                                        static_cast<Tp*>(out), static_cast<const Tp*>(x), weight,
                                        eps, H, x_stride, out_stride));
  return kvc_check_launch("kvc_rmsnorm");
}

template <typename T>
__global__ void residual_add_kernel(float* __restrict__ residual, const T* __restrict__ delta,
                                    int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) residual[i] += to_float(delta[i]);
}

extern "C" int kvc_residual_add(float* residual, const void* delta, int T, int H, int dtype,
                                kvc_stream stream) {
  if (T < 0 || H <= 0) return kvc_fail("kvc_residual_add: bad sizes");
  const int64_t n = static_cast<int64_t>(T) * H;
  if (n == 0) return 0;
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
  KVC_DISPATCH_DTYPE(dtype, Tp,
                     hipLaunchKernelGGL(residual_add_kernel<Tp>, dim3(blocks), dim3(256), 0,
                                        S(stream), residual, static_cast<const Tp*>(delta), n));
  return kvc_check_launch("kvc_residual_add");
}

// ------------------------------------------------------------------------- SiLU-mul
template <typename T>
__global__ void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gate_up, int I,
                                int64_t n) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  const int64_t t = idx / I;
  const int i = static_cast<int>(idx - t * I);
  const T* row = gate_up + t * 2 * I;
  const float g = to_float(row[i]);
  const float u = to_float(row[I + i]);
  const float s = g / (1.f + expf(-g));
  out[idx] = from_float<T>(s * u);
}

template <typename T>
__global__ void silu_mul_vec_kernel(T* __restrict__ out, const T* __restrict__ gate_up, int I8,
                                    int64_t n8) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n8) return;
  const int64_t t = idx / I8;
  const int64_t i = (idx - t * I8) * 8;
  const int64_t I = static_cast<int64_t>(I8) * 8;
  float g[8], u[8], y[8];
  load8(gate_up + t * 2 * I + i, g);
  load8(gate_up + t * 2 * I + I + i, u);
#pragma unroll
  for (int e = 0; e < 8; ++e) y[e] = g[e] / (1.f + expf(-g[e])) * u[e];
  store8(out + t * I + i, y);
}

extern "C" int kvc_silu_mul(void* out, const void* gate_up, int T, int I, int dtype,
                            kvc_stream stream) {
  if (T < 0 || I <= 0) return kvc_fail("kvc_silu_mul: bad sizes");
  const int64_t n = static_cast<int64_t>(T) * I;
  if (n == 0) return 0;
  if (I % 8 == 0 && (reinterpret_cast<uintptr_t>(out) % 16) == 0 &&
      (reinterpret_cast<uintptr_t>(gate_up) % 16) == 0) {
    const int64_t n8 = n / 8;
    const unsigned vblocks = static_cast<unsigned>((n8 + 255) / 256);
    KVC_DISPATCH_DTYPE(dtype, Tp,
                       hipLaunchKernelGGL(silu_mul_vec_kernel<Tp>, dim3(vblocks), dim3(256), 0,
                                          S(stream), static_cast<Tp*>(out),
                                          static_cast<const Tp*>(gate_up), I / 8, n8));
    return kvc_check_launch("kvc_silu_mul");
  }
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
  KVC_DISPATCH_DTYPE(dtype, Tp,
                     hipLaunchKernelGGL(silu_mul_kernel<Tp>, dim3(blocks), dim3(256), 0, S(stream),
                                        static_cast<Tp*>(out), static_cast<const Tp*>(gate_up), I,
                                        n));
  return kvc_check_launch("kvc_silu_mul");
}

// ----------------------------------------------------------------------- row gather
template <typename TI, typename TO>
__global__ void gather_rows_kernel(TO* __restrict__ out, const TI* __restrict__ in,
                                   const int32_t* __restrict__ rows, int H) {
  const int s = blockIdx.x;
  const TI* src = in + static_cast<int64_t>(rows[s]) * H;
  TO* dst = out + static_cast<int64_t>(s) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = from_float<TO>(to_float(src[i]));
}

extern "C" int kvc_gather_rows(void* out, const void* in, const int32_t* rows, int S_, int H,
                               int in_dtype, int out_dtype, kvc_stream stream) {
  if (S_ < 0 || H <= 0) return kvc_fail("kvc_gather_rows: bad sizes");
  if (S_ == 0) return 0;
  if (in_dtype == 0 && out_dtype == 0) {
    hipLaunchKernelGGL((gather_rows_kernel<float, float>), dim3(S_), dim3(256), 0, S(stream),
                       static_cast<float*>(out), static_cast<const float*>(in), rows, H);
  } else if (in_dtype == 1 && out_dtype == 1) {
    hipLaunchKernelGGL((gather_rows_kernel<bf16_t, bf16_t>), dim3(S_), dim3(256), 0, S(stream),
                       static_cast<bf16_t*>(out), static_cast<const bf16_t*>(in), rows, H);
  } else if (in_dtype == 0 && out_dtype == 1) {
    hipLaunchKernelGGL((gather_rows_kernel<float, bf16_t>), dim3(S_), dim3(256), 0, S(stream),
                       static_cast<bf16_t*>(out), static_cast<const float*>(in), rows, H);
  } else if (in_dtype == 1 && out_dtype == 0) {
    hipLaunchKernelGGL((gather_rows_kernel<bf16_t, float>), dim3(S_), dim3(256), 0, S(stream),
                       static_cast<float*>(out), static_cast<const bf16_t*>(in), rows, H);
  } else {
    return kvc_fail("kvc_gather_rows: unknown dtype code");
  }
  return kvc_check_launch("kvc_gather_rows");
}

template <typename T>
__global__ void to_float_kernel(float* __restrict__ out, const T* __restrict__ in, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) out[i] = to_float(in[i]);
}

extern "C" int kvc_to_float(float* out, const void* in, int64_t n, int dtype, kvc_stream stream) {
  if (n < 0) return kvc_fail("kvc_to_float: bad size");
  if (n == 0) return 0;
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
  KVC_DISPATCH_DTYPE(dtype, Tp,
                     hipLaunchKernelGGL(to_float_kernel<Tp>, dim3(blocks), dim3(256), 0, S(stream),
                                        out, static_cast<const Tp*>(in), n));
  return kvc_check_launch("kvc_to_float");
}

// -------------------------------------------------------------------- rotary tables
__global__ void rope_table_kernel(float* __restrict__ cos_out, float* __restrict__ sin_out,
                                  const int32_t* __restrict__ positions,
                                  const float* __restrict__ inv_freq, int half, int64_t n) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= n) return;
  const int64_t t = idx / half;
  const int j = static_cast<int>(idx - t * half);
  const float angle = static_cast<float>(positions[t]) * inv_freq[j];
  float s, c;
  sincosf(angle, &s, &c);
  cos_out[idx] = c;
  sin_out[idx] = s;
}

extern "C" int kvc_rope_table(float* cos_out, float* sin_out, const int32_t* positions,
                              const float* inv_freq, int T, int half, kvc_stream stream) {
  if (T < 0 || half <= 0) return kvc_fail("kvc_rope_table: bad sizes");
  const int64_t n = static_cast<int64_t>(T) * half;
  if (n == 0) return 0;
  const unsigned blocks = static_cast<unsigned>((n + 255) / 256);
  hipLaunchKernelGGL(rope_table_kernel, dim3(blocks), dim3(256), 0, S(stream), cos_out, sin_out,
                     positions, inv_freq, half, n);
  return kvc_check_launch("kvc_rope_table");
}

// ------------------------------------------------------------------ cache slots
// kv_slot[t] = page * page_size + position % page_size of token t in its request's block
// table row; -1 when the table has no page there; -2 for a padding token.
__global__ void kv_slots_kernel(int32_t* __restrict__ kv_slot, const int32_t* __restrict__ positions,
                                const int32_t* __restrict__ token_req,
                                const int32_t* __restrict__ slots, const int32_t* __restrict__ table,
                                int table_stride, int T, int page_size, int num_pages) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const int req = token_req[t];
  if (req < 0) {
    kv_slot[t] = -2;
    return;
  }
  const int pos = positions[t];
  const int idx = pos / page_size;
  int out = -1;
  if (idx < table_stride) {
    const int page = table[static_cast<int64_t>(slots[req]) * table_stride + idx];
    if (page > 0 && page < num_pages) out = page * page_size + pos % page_size;
  }
  kv_slot[t] = out;
}

extern "C" int kvc_kv_slots(int32_t* kv_slot, const int32_t* positions, const int32_t* token_req,
                            const int32_t* slots, const int32_t* table, int table_stride, int T,
                            int page_size, int num_pages, kvc_stream stream) {
  if (T < 0 || table_stride <= 0 || page_size <= 0 || num_pages <= 0)
    return kvc_fail("kvc_kv_slots: bad sizes");
  if (static_cast<int64_t>(num_pages) * page_size > 0x7fffffffLL)
    return kvc_fail("kvc_kv_slots: cache too large for 32-bit slots");
  if (T == 0) return 0;
  hipLaunchKernelGGL(kv_slots_kernel, dim3((T + 255) / 256), dim3(256), 0, S(stream), kv_slot,
                     positions, token_req, slots, table, table_stride, T, page_size, num_pages);
  return kvc_check_launch("kvc_kv_slots");
}

// ------------------------------------------------- rotation fused with the K/V write
// One block per token.  Work items: (head, pair) rotations for the nh + nkv rotated
// heads, then pass-through elements (beyond rot_dim, and all of v).  K pages are
// [kv head, page_size, d]; V pages are [kv head, d, page_size] (keys contiguous).
// VEC = 8 handles eight pairs per item with 16-byte accesses (half-split pairing, rot_dim
// a multiple of 16); VEC = 1 is the general path.
template <typename T, int VEC>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, T* __restrict__ k_cache,
                                     T* __restrict__ v_cache, const float* __restrict__ cos_tab,
                                     const float* __restrict__ sin_tab, int rot_dim,
                                     int interleaved, const int32_t* __restrict__ kv_slot, int nh,
                                     int nkv, int d, int page_size, int write_kv, int head_begin) {
  const int t = blockIdx.x;
  const int slot = kv_slot[t];
  if (slot == -2) return;  // padding token
  const int half = rot_dim / 2;
  T* row = qkv + static_cast<int64_t>(t) * (nh + 2 * nkv) * d;

  int64_t k_base = -1, v_base = -1;
  if (write_kv && slot >= 0) {
    const int page = slot / page_size, off = slot - page * page_size;
    k_base = (static_cast<int64_t>(page) * nkv * page_size + off) * d;       // K[page, 0, off, 0]
    v_base = static_cast<int64_t>(page) * nkv * page_size * d + off;         // V[page, 0, 0, off]
  }
  const int64_t head_step = static_cast<int64_t>(page_size) * d;  // between kv heads in a page
  const float* cs = cos_tab + static_cast<int64_t>(t) * half;
  const float* sn = sin_tab + static_cast<int64_t>(t) * half;

  if constexpr (VEC == 8) {
    const int chunks = half / 8;
    const int n_items = (nh + nkv - head_begin) * chunks;  // head_begin = nh: the keys only
    for (int w = threadIdx.x; w < n_items; w += blockDim.x) {
      const int head = head_begin + w / chunks;
      const int j = (w - (head - head_begin) * chunks) * 8;
      T* hp = row + static_cast<int64_t>(head) * d;
      float x0[8], x1[8], c[8], s_[8], y0[8], y1[8];
      load8(hp + j, x0);
      load8(hp + j + half, x1);
      load8(cs + j, c);
      load8(sn + j, s_);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        y0[e] = rotate_first(x0[e], x1[e], c[e], s_[e]);
        y1[e] = rotate_second(x0[e], x1[e], c[e], s_[e]);
      }
      store8(hp + j, y0);
      store8(hp + j + half, y1);
      if (head >= nh && k_base >= 0) {
        T* kc = k_cache + k_base + (head - nh) * head_step;
        store8(kc + j, y0);
        store8(kc + j + half, y1);
      }
    }
  } else {
    const int n_rot = (nh + nkv - head_begin) * half;
    for (int w = threadIdx.x; w < n_rot; w += blockDim.x) {
      const int head = head_begin + w / half;
      const int j = w - (head - head_begin) * half;
      const int i0 = interleaved ? 2 * j : j;
      const int i1 = interleaved ? 2 * j + 1 : j + half;
      T* hp = row + static_cast<int64_t>(head) * d;
      const float x0 = to_float(hp[i0]);
      const float x1 = to_float(hp[i1]);
      const float c = cs[j], s_ = sn[j];
      const T y0 = from_float<T>(rotate_first(x0, x1, c, s_));
      const T y1 = from_float<T>(rotate_second(x0, x1, c, s_));
      hp[i0] = y0;
      hp[i1] = y1;
      if (head >= nh && k_base >= 0) {
        T* kc = k_cache + k_base + (head - nh) * head_step;
        kc[i0] = y0;
        kc[i1] = y1;
      }
    }
  }
  if (k_base < 0) return;
  // k elements beyond the rotated part
  const int tail = d - rot_dim;
  if (tail > 0) {
    for (int w = threadIdx.x; w < nkv * tail; w += blockDim.x) {
      const int head = w / tail;
      const int i = rot_dim + (w - head * tail);
      k_cache[k_base + head * head_step + i] = row[static_cast<int64_t>(nh + head) * d + i];
    }
  }
  // v, element i of a head goes to V[page, head, i, off]
  for (int w = threadIdx.x; w < nkv * d; w += blockDim.x) {
    const int head = w / d;
    const int i = w - head * d;
    v_cache[v_base + head * head_step + static_cast<int64_t>(i) * page_size] =
        row[static_cast<int64_t>(nh + nkv + head) * d + i];
  }
}

// The same for eight consecutive tokens a block, with 16-byte accesses throughout (half-split
// pairing, rot_dim a multiple of 16, head size a multiple of 8).  A V page keeps the keys
// contiguous, so a token alone stores its value two bytes at a time, d * nkv stores 32 bytes
// apart; when the block's eight tokens lie side by side in one page (a portion of a prompt
// mostly does), a thread gathers one element of all eight and stores them together.
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_tile_kernel(
    T* __restrict__ qkv, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const float* __restrict__ cos_tab, const float* __restrict__ sin_tab, int rot_dim,
    const int32_t* __restrict__ kv_slot, int num_tokens, int nh, int nkv, int d, int page_size,
    int write_kv, int head_begin) {
  constexpr int TILE = 8;
  const int t0 = blockIdx.x * TILE;
  const int n_tok = (num_tokens - t0 < TILE) ? num_tokens - t0 : TILE;
  const int half = rot_dim / 2;
  const int64_t row_elems = static_cast<int64_t>(nh + 2 * nkv) * d;
  const int64_t head_step = static_cast<int64_t>(page_size) * d;  // between kv heads in a page
  const int chunks = half / 8;
  const int n_items = (nh + nkv - head_begin) * chunks;  // head_begin = nh: the keys only
  // ---- rotations, and the rotated keys into the cache
  for (int w = threadIdx.x; w < n_tok * n_items; w += blockDim.x) {
    const int ti = w / n_items;
    const int item = w - ti * n_items;
    const int t = t0 + ti;
    const int slot = kv_slot[t];
    if (slot == -2) continue;  // padding token
    const int head = head_begin + item / chunks;
    const int j = (item - (head - head_begin) * chunks) * 8;
    T* hp = qkv + t * row_elems + static_cast<int64_t>(head) * d;
    const float* cs = cos_tab + static_cast<int64_t>(t) * half;
    const float* sn = sin_tab + static_cast<int64_t>(t) * half;
    float x0[8], x1[8], c[8], s_[8], y0[8], y1[8];
    load8(hp + j, x0);
    load8(hp + j + half, x1);
    load8(cs + j, c);
    load8(sn + j, s_);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      y0[e] = rotate_first(x0[e], x1[e], c[e], s_[e]);
      y1[e] = rotate_second(x0[e], x1[e], c[e], s_[e]);
    }
    store8(hp + j, y0);
    store8(hp + j + half, y1);
    if (head >= nh && write_kv && slot >= 0) {
      const int page = slot / page_size, off = slot - page * page_size;
      T* kc = k_cache + (static_cast<int64_t>(page) * nkv * page_size + off) * d + (head - nh) * head_step;
      store8(kc + j, y0);
      store8(kc + j + half, y1);
    }
  }
  if (!write_kv) return;
  // ---- k elements beyond the rotated part, eight at a time
  const int tail_chunks = (d - rot_dim) / 8;
  for (int w = threadIdx.x; w < n_tok * nkv * tail_chunks; w += blockDim.x) {
    const int ti = w / (nkv * tail_chunks);
    const int rest = w - ti * nkv * tail_chunks;
    const int head = rest / tail_chunks;
    const int i = rot_dim + (rest - head * tail_chunks) * 8;
    const int slot = kv_slot[t0 + ti];
    if (slot < 0) continue;
    const int page = slot / page_size, off = slot - page * page_size;
    float v[8];
    load8(qkv + (t0 + ti) * row_elems + static_cast<int64_t>(nh + head) * d + i, v);
    store8(k_cache + (static_cast<int64_t>(page) * nkv * page_size + off) * d + head * head_step + i, v);
  }
  // ---- v: element i of a head goes to V[page, head, i, off]
  const int s0 = kv_slot[t0];
  bool side_by_side = n_tok == TILE && s0 >= 0 && (s0 & 7) == 0 && (page_size & 7) == 0;
  for (int ti = 1; ti < n_tok; ++ti) side_by_side = side_by_side && kv_slot[t0 + ti] == s0 + ti;
  // (eight slots from a multiple of eight stay within a page whose size is a multiple of eight)
  if (side_by_side) {
    const int page = s0 / page_size, off = s0 - page * page_size;
    const int64_t v_base = static_cast<int64_t>(page) * nkv * page_size * d + off;
    for (int w = threadIdx.x; w < nkv * d; w += blockDim.x) {
      const int head = w / d;
      const int i = w - head * d;
      const T* src = qkv + t0 * row_elems + static_cast<int64_t>(nh + nkv + head) * d + i;
      alignas(16) T vals[TILE];
#pragma unroll
      for (int ti = 0; ti < TILE; ++ti) vals[ti] = src[ti * row_elems];
      T* dst = v_cache + v_base + head * head_step + static_cast<int64_t>(i) * page_size;
      if constexpr (sizeof(T) == 2) {
        *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(vals);
      } else {
        *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(vals);
        *reinterpret_cast<uint4*>(dst + 4) = *reinterpret_cast<const uint4*>(vals + 4);
      }
    }
    return;
  }
  for (int w = threadIdx.x; w < n_tok * nkv * d; w += blockDim.x) {
    const int ti = w / (nkv * d);
    const int rest = w - ti * nkv * d;
    const int head = rest / d;
    const int i = rest - head * d;
    const int slot = kv_slot[t0 + ti];
    if (slot < 0) continue;
    const int page = slot / page_size, off = slot - page * page_size;
    v_cache[static_cast<int64_t>(page) * nkv * page_size * d + off + head * head_step +
            static_cast<int64_t>(i) * page_size] =
        qkv[(t0 + ti) * row_elems + static_cast<int64_t>(nh + nkv + head) * d + i];
  }
}

extern "C" int kvc_rope_kv_write(void* qkv, void* k_cache, void* v_cache, const float* cos_tab,
                                 const float* sin_tab, int rot_dim, int interleaved,
                                 const int32_t* kv_slot, int T, int nh, int nkv, int d,
                                 int page_size, int write_kv, int rotate_q, int dtype,
                                 kvc_stream stream) {
  if (T < 0 || nh <= 0 || nkv <= 0 || d <= 0 || page_size <= 0)
    return kvc_fail("kvc_rope_kv_write: bad sizes");
  const int head_begin = rotate_q ? 0 : nh;
  if (rot_dim < 0 || rot_dim > d || (rot_dim & 1))
    return kvc_fail("kvc_rope_kv_write: rot_dim must be even and at most the head size");
  if (T == 0) return 0;
  const auto aligned16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  const bool vec = !interleaved && rot_dim > 0 && rot_dim % 16 == 0 && d % 8 == 0 &&
                   aligned16(qkv) && aligned16(k_cache) && aligned16(cos_tab) && aligned16(sin_tab);
  if (vec && T >= 16 && aligned16(v_cache)) {
    // steps of many tokens: eight tokens a block
    kvc_note_variant(kVariantRopeKvWrite, "rope_kv_write_tile_kernel");
    KVC_DISPATCH_DTYPE(
        dtype, Tp,
        hipLaunchKernelGGL((rope_kv_write_tile_kernel<Tp>), dim3((T + 7) / 8), dim3(256), 0, S(stream),
                           static_cast<Tp*>(qkv), static_cast<Tp*>(k_cache),
                           static_cast<Tp*>(v_cache), cos_tab, sin_tab, rot_dim, kv_slot, T, nh, nkv, d,
                           page_size, write_kv, head_begin));
  } else if (vec) {
    kvc_note_variant(kVariantRopeKvWrite, "rope_kv_write_kernel<8>");
    KVC_DISPATCH_DTYPE(
        dtype, Tp,
        hipLaunchKernelGGL((rope_kv_write_kernel<Tp, 8>), dim3(T), dim3(256), 0, S(stream),
                           static_cast<Tp*>(qkv), static_cast<Tp*>(k_cache),
                           static_cast<Tp*>(v_cache), cos_tab, sin_tab, rot_dim, interleaved,
                           kv_slot, nh, nkv, d, page_size, write_kv, head_begin));
  } else {
    kvc_note_variant(kVariantRopeKvWrite, "rope_kv_write_kernel<1>");
    KVC_DISPATCH_DTYPE(
        dtype, Tp,
        hipLaunchKernelGGL((rope_kv_write_kernel<Tp, 1>), dim3(T), dim3(256), 0, S(stream),
                           static_cast<Tp*>(qkv), static_cast<Tp*>(k_cache),
                           static_cast<Tp*>(v_cache), cos_tab, sin_tab, rot_dim, interleaved,
                           kv_slot, nh, nkv, d, page_size, write_kv, head_begin));
  }
  return kvc_check_launch("kvc_rope_kv_write");
}

// ------------------------------------------------------------- block-table updates
__global__ void table_update_kernel(int32_t* __restrict__ table, int table_stride, int table_rows,
                                    const int32_t* __restrict__ triples, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int row = triples[3 * i], col = triples[3 * i + 1], val = triples[3 * i + 2];
  if (row < 0 || row >= table_rows || col < 0 || col >= table_stride) return;
  table[static_cast<int64_t>(row) * table_stride + col] = val;
}

extern "C" int kvc_table_update(int32_t* table, int table_stride, int table_rows,
                                const int32_t* triples, int n, kvc_stream stream) {
  if (n < 0 || table_stride <= 0 || table_rows <= 0) return kvc_fail("kvc_table_update: bad sizes");
  if (n == 0) return 0;
  hipLaunchKernelGGL(table_update_kernel, dim3((n + 255) / 256), dim3(256), 0, S(stream), table,
                     table_stride, table_rows, triples, n);
  return kvc_check_launch("kvc_table_update");
}
