// C ABI of libtpumlir_amd.so: operator-level entry points (float-expanded host operands, as the reference
// interpreter hands them over) and device-level launches.  See include/tpumlir_amd.h for the contract.
#include <math.h>
#if defined(__SSE2__)
#include <immintrin.h>
#endif
#include <string.h>

#include <algorithm>
#include <new>
#include <string>
#include <vector>

#include <atomic>

#include "internal.h"

namespace mi {

static thread_local std::string g_last_error;
// The override record is published as a pointer to an immutable copy, so a launch on one thread reads either the old
// record or the new one, never a mixture.  Superseded copies are not freed (a launch may still be reading one); the hook
// is a test and tuning aid, called a handful of times per process.
static const mi_internal_plan g_no_plan = {};
static std::atomic<const mi_internal_plan *> g_plan{&g_no_plan};

const mi_internal_plan &plan() { return *g_plan.load(std::memory_order_acquire); }

void set_error(const std::string &msg) { g_last_error = msg; }

int hip_fail(hipError_t e, const char *what, const char *file, int line) {
  g_last_error = std::string("HIP error ") + hipGetErrorName(e) + " (" + hipGetErrorString(e) + ") in " + what +
                 " at " + file + ":" + std::to_string(line);
  (void)hipGetLastError();  // clear the sticky error so that the next call reports its own
  return MI_HIP_ERROR;
}

static inline uint32_t fbits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float bits_f(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}

// host-side f32 <-> 16-bit conversions used only to stage interpreter tensors (values that already are
// bf16/f16 numbers convert exactly; anything else is rounded to nearest even)
static inline uint16_t h_f32_to_bf16(float f) {
  uint32_t u = fbits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u)
    return 0x7fff;
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
static inline float h_bf16_to_f32(uint16_t h) { return bits_f((uint32_t)h << 16); }
static inline uint16_t h_f32_to_f16(float f) {
  _Float16 h = (_Float16)f;
  uint16_t b;
  memcpy(&b, &h, 2);
  return (f != f) ? (uint16_t)0x7fff : b;
}
static inline float h_f16_to_f32(uint16_t b) {
  _Float16 h;
  memcpy(&h, &b, 2);
  return (float)h;
}

// pinned host staging buffer that only grows
struct Pinned {
  void *ptr = nullptr;
  size_t cap = 0;
  int reserve(size_t bytes) {
    if (bytes <= cap)
      return MI_SUCCESS;
    if (ptr)
      (void)hipHostFree(ptr);
    ptr = nullptr;
    cap = 0;
    MI_HIP(hipHostMalloc(&ptr, bytes, hipHostMallocDefault));
    cap = bytes;
    return MI_SUCCESS;
  }
  ~Pinned() {
    if (ptr)
      (void)hipHostFree(ptr);
  }
};

struct DevBuf {
  void *ptr = nullptr;
  size_t cap = 0;
  int reserve(size_t bytes) {
    if (bytes <= cap)
      return MI_SUCCESS;
    if (ptr)
      (void)hipFree(ptr);
    ptr = nullptr;
    cap = 0;
    MI_HIP(hipMalloc(&ptr, bytes));
    cap = bytes;
    return MI_SUCCESS;
  }
  ~DevBuf() {
    if (ptr)
      (void)hipFree(ptr);
  }
};

// ---------------------------------------------------------------------------------------------
// tpu.A16MatMul operator state
// ---------------------------------------------------------------------------------------------
// The interpreter's tensors are f32 arrays; the matmul wants 16-bit operands.  These two kernels convert on the device
// (the same rounding as h_f32_to_bf16 / h_f32_to_f16), so that a call costs no host loop over the elements.  For a
// small call `in` / `out` are pinned host buffers read and written over the bus by the kernel itself, which saves the
// two copy commands and their latency.
__global__ __launch_bounds__(256) void stage_f32_to_16_kernel(const float *in, uint16_t *out, int64_t n, int f16) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const float f = in[i];
    const uint32_t u = __builtin_bit_cast(uint32_t, f);
    uint16_t h;
    if ((u & 0x7fffffffu) > 0x7f800000u)
      h = 0x7fff;
    else if (f16)
      h = __builtin_bit_cast(uint16_t, (_Float16)f);
    else
      h = (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
    out[i] = h;
  }
}
__global__ __launch_bounds__(256) void expand_16_to_f32_kernel(const uint16_t *in, float *out, int64_t n, int f16) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const uint16_t h = in[i];
    out[i] = f16 ? (float)__builtin_bit_cast(_Float16, h) : __builtin_bit_cast(float, (uint32_t)h << 16);
  }
}
static unsigned stage_grid(int64_t n) {
  int64_t b = (n + 255) / 256;
  return (unsigned)(b > 4096 ? 4096 : b);
}
// calls with at most this many elements on a side go through the pinned buffers
constexpr int64_t SMALL_CALL_ELEMS = 1 << 16;
// the quantized MatMul's 8-bit operand and its result travel the same way up to this many bytes
constexpr size_t SMALL_I8_CALL_BYTES = (size_t)1 << 20;
__global__ __launch_bounds__(256) void copy16_kernel(const uint4 *in, uint4 *out, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
    out[i] = in[i];
}

struct A16Handle {
  uint32_t magic = 0xA16A16u;
  mi_a16_weight *w = nullptr;
  Pinned h_x, h_y;             // small calls: f32 activations in, 16-bit results out, both touched by the kernels directly
  DevBuf d_x, d_y, d_xf, d_yf; // 16-bit operands of the matmul; f32 staging of large calls
  hipStream_t stream = nullptr;
  ~A16Handle() {
    if (w) {
      a16_free(w);
      delete w;
    }
    if (stream) {
      release_stream_workspaces(stream);
      (void)hipStreamDestroy(stream);
    }
  }
};

static bool group_size_supported(int bits, int g, int64_t K) {
  if (g == 0)
    return true;
  if (g < 0 || K % g != 0)
    return false;
  if (bits == 4)
    return g == 32 || g == 64 || (g % W4_TILE_K) == 0;
  return g == 32 || (g % W8_TILE_K) == 0;
}

}  // namespace mi

using namespace mi;

extern "C" {

void mi_internal_set_plan(const mi_internal_plan *p) {
  g_plan.store(p ? new mi_internal_plan(*p) : &g_no_plan, std::memory_order_release);
}
long mi_internal_workspace_allocations(void) { return mi::workspace_allocations(); }

const char *mi_version(void) { return "tpumlir_amd 0.1 (gfx950)"; }
const char *mi_last_error(void) { return g_last_error.c_str(); }

int mi_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  return n;
}

// ---------------------------------------------------------------------------------------------
// device level: A16 weights
// ---------------------------------------------------------------------------------------------
int mi_a16_weight_create(mi_a16_weight **out, const mi_a16_weight_desc *d, const void *weight,
                         const uint16_t *scale, const uint8_t *zp, const float *bias) {
  MI_REQUIRE(out && d && weight && scale && zp, MI_BAD_ARGUMENT, "mi_a16_weight_create: null argument");
  *out = nullptr;
  MI_REQUIRE(d->weight_bits == 4 || d->weight_bits == 8, MI_UNSUPPORTED,
             "mi_a16_weight_create: weight_bits must be 4 or 8");
  MI_REQUIRE(d->dtype == MI_DT_BF16 || d->dtype == MI_DT_F16, MI_UNSUPPORTED,
             "mi_a16_weight_create: dtype must be bf16 or f16");
  MI_REQUIRE(d->K > 0 && d->N > 0, MI_BAD_ARGUMENT, "mi_a16_weight_create: bad shape");
  MI_REQUIRE(d->K % 8 == 0, MI_UNSUPPORTED, "mi_a16_weight_create: K must be a multiple of 8");
  MI_REQUIRE(d->q_group_size == 0 || (d->q_group_size > 0 && d->K % d->q_group_size == 0), MI_BAD_ARGUMENT,
             "mi_a16_weight_create: K is not a multiple of q_group_size");
  MI_REQUIRE(mi_device_count() > 0, MI_HIP_ERROR, "mi_a16_weight_create: no GPU visible");
  mi_a16_weight *w = new (std::nothrow) mi_a16_weight();
  MI_REQUIRE(w, MI_HIP_ERROR, "mi_a16_weight_create: out of host memory");
  w->K = d->K;
  w->N = d->N;
  w->bits = d->weight_bits;
  w->g = d->q_group_size;
  w->G = d->q_group_size ? (int)(d->K / d->q_group_size) : 1;
  w->dtype = d->dtype;
  w->chip = d->chip;
  // group sizes of 32, 64 or whole k-tiles are packed for the tiled kernels; any other stays as stored (a16_plain.hip)
  int rc = group_size_supported(d->weight_bits, d->q_group_size, d->K)
               ? a16_pack(w, weight, d->weight_signed, scale, zp, bias)
               : a16_plain_create(w, weight, d->weight_signed, scale, zp, bias);
  if (rc != MI_SUCCESS) {
    mi_a16_weight_destroy(w);
    return rc;
  }
  *out = w;
  return MI_SUCCESS;
}

void mi_a16_weight_destroy(mi_a16_weight *w) {
  if (!w)
    return;
  a16_free(w);
  delete w;
}

size_t mi_a16_weight_bytes(const mi_a16_weight *w) { return w ? w->bytes : 0; }

// ---- packed weight set <-> blob ---------------------------------------------------------------------------------
namespace {
struct BlobHeader {
  char magic[8];  // "MIA16W1\0"
  int64_t K, N, row_blocks, k_tiles;
  int32_t bits, g, G, dtype, chip, has_bias;
  uint64_t packed_bytes, qparam_entries;  // qparam_entries = row_blocks * G * 16
};
const char kBlobMagic[8] = {'M', 'I', 'A', '1', '6', 'W', '1', 0};
size_t blob_payload(const BlobHeader &h) {
  return (size_t)h.packed_bytes + (size_t)h.qparam_entries * (h.bits == 4 ? 4 : 6) + (h.has_bias ? (size_t)h.N * 4 : 0);
}
BlobHeader blob_header_of(const mi_a16_weight *w) {
  BlobHeader h;
  memset(&h, 0, sizeof(h));
  memcpy(h.magic, kBlobMagic, 8);
  h.K = w->K;
  h.N = w->N;
  h.row_blocks = w->row_blocks;
  h.k_tiles = w->k_tiles;
  h.bits = w->bits;
  h.g = w->g;
  h.G = w->G;
  h.dtype = w->dtype;
  h.chip = w->chip;
  h.has_bias = w->bias != nullptr;
  h.packed_bytes = (uint64_t)w->row_blocks * w->k_tiles * 1024;
  h.qparam_entries = (uint64_t)w->row_blocks * w->G * 16;
  return h;
}
}  // namespace

size_t mi_a16_weight_export_size(const mi_a16_weight *w) {
  if (!w)
    return 0;
  const BlobHeader h = blob_header_of(w);
  return sizeof(BlobHeader) + blob_payload(h);
}

int mi_a16_weight_export(const mi_a16_weight *w, void *blob, size_t capacity) {
  MI_REQUIRE(w && blob, MI_BAD_ARGUMENT, "mi_a16_weight_export: null argument");
  const BlobHeader h = blob_header_of(w);
  MI_REQUIRE(capacity >= sizeof(BlobHeader) + blob_payload(h), MI_BAD_ARGUMENT,
             "mi_a16_weight_export: buffer smaller than mi_a16_weight_export_size()");
  uint8_t *p = (uint8_t *)blob;
  memcpy(p, &h, sizeof(h));
  p += sizeof(h);
  MI_REQUIRE(!w->kn && !w->plain, MI_UNSUPPORTED,
             "mi_a16_weight_export: a weight kept as stored (untransposed, or a group size outside the tiled layout) "
             "has no packed form");
  MI_HIP(hipMemcpy(p, w->qweight, h.packed_bytes, hipMemcpyDeviceToHost));
  p += h.packed_bytes;
  if (w->bits == 4) {
    MI_HIP(hipMemcpy(p, w->sz_t, h.qparam_entries * 4, hipMemcpyDeviceToHost));
    p += h.qparam_entries * 4;
  } else {
    MI_HIP(hipMemcpy(p, w->scale_t, h.qparam_entries * 2, hipMemcpyDeviceToHost));
    p += h.qparam_entries * 2;
    MI_HIP(hipMemcpy(p, w->nzs_t, h.qparam_entries * 4, hipMemcpyDeviceToHost));
    p += h.qparam_entries * 4;
  }
  if (h.has_bias)
    MI_HIP(hipMemcpy(p, w->bias, (size_t)h.N * 4, hipMemcpyDeviceToHost));
  return MI_SUCCESS;
}

int mi_a16_weight_import(mi_a16_weight **out, const void *blob, size_t size) {
  MI_REQUIRE(out && blob, MI_BAD_ARGUMENT, "mi_a16_weight_import: null argument");
  *out = nullptr;
  MI_REQUIRE(size >= sizeof(BlobHeader), MI_BAD_ARGUMENT, "mi_a16_weight_import: truncated blob");
  BlobHeader h;
  memcpy(&h, blob, sizeof(h));
  MI_REQUIRE(memcmp(h.magic, kBlobMagic, 8) == 0, MI_BAD_ARGUMENT, "mi_a16_weight_import: not a packed A16 weight blob");
  MI_REQUIRE((h.bits == 4 || h.bits == 8) && h.K > 0 && h.N > 0 && h.G >= 1 &&
                 (h.dtype == MI_DT_BF16 || h.dtype == MI_DT_F16),
             MI_BAD_ARGUMENT, "mi_a16_weight_import: bad header");
  const int tile_k = h.bits == 4 ? mi::W4_TILE_K : mi::W8_TILE_K;
  MI_REQUIRE(h.row_blocks == (h.N + 15) / 16 && h.k_tiles == (h.K + tile_k - 1) / tile_k &&
                 h.packed_bytes == (uint64_t)h.row_blocks * h.k_tiles * 1024 &&
                 h.qparam_entries == (uint64_t)h.row_blocks * h.G * 16 && (h.g == 0 ? h.G == 1 : (int64_t)h.g * h.G == h.K),
             MI_BAD_ARGUMENT, "mi_a16_weight_import: header fields disagree with each other");
  MI_REQUIRE(group_size_supported(h.bits, h.g, h.K), MI_UNSUPPORTED, "mi_a16_weight_import: group size not handled");
  MI_REQUIRE(size == sizeof(BlobHeader) + blob_payload(h), MI_BAD_ARGUMENT, "mi_a16_weight_import: size mismatch");
  MI_REQUIRE(mi_device_count() > 0, MI_HIP_ERROR, "mi_a16_weight_import: no GPU visible");
  mi_a16_weight *w = new (std::nothrow) mi_a16_weight();
  MI_REQUIRE(w, MI_HIP_ERROR, "mi_a16_weight_import: out of host memory");
  w->K = h.K;
  w->N = h.N;
  w->bits = h.bits;
  w->g = h.g;
  w->G = h.G;
  w->dtype = h.dtype;
  w->chip = h.chip;
  w->row_blocks = h.row_blocks;
  w->k_tiles = h.k_tiles;
  const uint8_t *p = (const uint8_t *)blob + sizeof(h);
  auto upload = [&](void **dst, size_t bytes) -> int {
    MI_HIP(hipMalloc(dst, bytes));
    MI_HIP(hipMemcpy(*dst, p, bytes, hipMemcpyHostToDevice));
    p += bytes;
    w->bytes += bytes;
    return MI_SUCCESS;
  };
  int rc = upload(&w->qweight, h.packed_bytes);
  if (rc == MI_SUCCESS && h.bits == 4)
    rc = upload((void **)&w->sz_t, h.qparam_entries * 4);
  if (rc == MI_SUCCESS && h.bits == 8)
    rc = upload((void **)&w->scale_t, h.qparam_entries * 2);
  if (rc == MI_SUCCESS && h.bits == 8)
    rc = upload((void **)&w->nzs_t, h.qparam_entries * 4);
  if (rc == MI_SUCCESS && h.has_bias)
    rc = upload((void **)&w->bias, (size_t)h.N * 4);
  if (rc == MI_SUCCESS)
    rc = a16_build_sz_dec(w);
  if (rc != MI_SUCCESS) {
    a16_free(w);
    delete w;
    return rc;
  }
  *out = w;
  return MI_SUCCESS;
}

// ---- weight producers ----------------------------------------------------------------------------------------
int mi_a16_quantize(const mi_a16_quant_desc *d, const float *w_kn, void *weight, uint16_t *scale16, float *scale_f32,
                    uint8_t *zp, int *sign, int *weight_signed) {
  MI_REQUIRE(d && w_kn && weight && scale16 && zp, MI_BAD_ARGUMENT, "mi_a16_quantize: null argument");
  MI_REQUIRE(d->weight_bits == 4 || d->weight_bits == 8, MI_UNSUPPORTED, "mi_a16_quantize: weight_bits must be 4 or 8");
  MI_REQUIRE(d->dtype == MI_DT_BF16 || d->dtype == MI_DT_F16, MI_UNSUPPORTED, "mi_a16_quantize: dtype must be bf16 or f16");
  MI_REQUIRE(d->K > 0 && d->N > 0 && (d->weight_bits == 8 || d->K % 2 == 0), MI_BAD_ARGUMENT, "mi_a16_quantize: bad shape");
  const int64_t gs = d->q_group_size == -1 ? d->K : d->q_group_size;
  MI_REQUIRE(gs >= 0 && (gs == 0 || d->K % gs == 0), MI_BAD_ARGUMENT, "mi_a16_quantize: K is not a multiple of q_group_size");
  MI_REQUIRE(gs == 0 || d->K / gs <= 65535, MI_UNSUPPORTED, "mi_a16_quantize: more than 65535 groups per row");
  MI_REQUIRE(d->dq_type == MI_DQ_NONE || d->dq_type == MI_DQ_INT ||
                 (gs != 0 && ((d->dq_type == MI_DQ_F8E4M3 && d->weight_bits == 8) ||
                              (d->dq_type == MI_DQ_F4 && d->weight_bits == 4))),
             MI_UNSUPPORTED, "mi_a16_quantize: float code types need groups, F8E4M3 8-bit and F4 4-bit weights");
  MI_REQUIRE(!d->zp_float || d->dq_type == MI_DQ_NONE || d->dq_type == MI_DQ_INT, MI_UNSUPPORTED,
             "mi_a16_quantize: float zero points go with integer codes only");
  MI_REQUIRE(mi_device_count() > 0, MI_HIP_ERROR, "mi_a16_quantize: no GPU visible");
  return a16_quantize(d, w_kn, weight, scale16, scale_f32, zp, sign, weight_signed);
}

int mi_llm_unpack(int mode, int bits, const int32_t *qweight, const int32_t *qzeros, int64_t K, int64_t N, int64_t G,
                  uint8_t *weight, uint8_t *zp) {
  MI_REQUIRE(qweight && qzeros && weight && zp, MI_BAD_ARGUMENT, "mi_llm_unpack: null argument");
  MI_REQUIRE(mode == MI_PACK_GPTQ || mode == MI_PACK_AWQ, MI_BAD_ARGUMENT, "mi_llm_unpack: mode");
  MI_REQUIRE(bits == 4 || (bits == 8 && mode == MI_PACK_GPTQ), MI_UNSUPPORTED,
             "mi_llm_unpack: 4-bit, or 8-bit GPTQ");
  const int ratio = 32 / bits;
  MI_REQUIRE(K > 0 && N > 0 && G > 0 && K % ratio == 0 && N % ratio == 0 && K % 2 == 0, MI_BAD_ARGUMENT,
             "mi_llm_unpack: K and N must be multiples of the values per int32");
  MI_REQUIRE(G <= 65535 && (bits == 4 ? K / 2 : K) <= 65535, MI_UNSUPPORTED, "mi_llm_unpack: shape too large");
  MI_REQUIRE(mi_device_count() > 0, MI_HIP_ERROR, "mi_llm_unpack: no GPU visible");
  return llm_unpack(mode, bits, qweight, qzeros, K, N, G, weight, zp);
}

// A16MatMulToGroup (Canonicalize/A16MatMul.cpp:432-499): per-channel parameters repeated K / 128 times along a new
// group axis, after which the op carries q_group_size 128.  Tiny host arrays: no kernel.
int mi_a16_to_group(const uint16_t *scale, int64_t scale_num, const uint8_t *zp, int64_t zp_num, int64_t K,
                    uint16_t *scale_out, uint8_t *zp_out) {
  MI_REQUIRE(scale && zp && scale_out && zp_out && scale_num > 0 && zp_num > 0, MI_BAD_ARGUMENT,
             "mi_a16_to_group: null argument");
  MI_REQUIRE(K >= 128 && K % 128 == 0, MI_UNSUPPORTED, "mi_a16_to_group: K must be a multiple of 128");
  const int64_t tile = K / 128;  // :460-461
  for (int64_t i = 0; i < scale_num; ++i)
    for (int64_t j = 0; j < tile; ++j)
      scale_out[i * tile + j] = scale[i];
  for (int64_t i = 0; i < zp_num; ++i)
    for (int64_t j = 0; j < tile; ++j)
      zp_out[i * tile + j] = zp[i];
  return MI_SUCCESS;
}

int mi_a16mm_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y_f32,
                    void *stream) {
  return a16_launch(w, d_x, M, d_y, d_y_f32, (hipStream_t)stream);
}

int mi_a16mm_dq_launch(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y_f32,
                       void *stream) {
  return a16_dq_launch(w, MI_DQ_INT, d_x, M, d_y, d_y_f32, (hipStream_t)stream);
}

int mi_a16mm_dq_type_launch(const mi_a16_weight *w, int dq_type, const uint16_t *d_x, int64_t M, uint16_t *d_y,
                            float *d_y_f32, void *stream) {
  return a16_dq_launch(w, dq_type, d_x, M, d_y, d_y_f32, (hipStream_t)stream);
}

int mi_a16mm_launch_tol(const mi_a16_weight *w, const uint16_t *d_x, int64_t M, uint16_t *d_y, float *d_y_f32,
                        void *stream) {
  MI_REQUIRE(w, MI_BAD_ARGUMENT, "mi_a16mm_launch_tol: null weight set");
  return a16_tol_launch(w, d_x, M, d_y, d_y_f32, (hipStream_t)stream);
}

int mi_a16mm_launch_group(const mi_a16_weight *const *w, int n, const uint16_t *d_x, int64_t M, uint16_t *const *d_y,
                          float *const *d_y_f32, void *stream) {
  return a16_launch_group(w, n, d_x, M, d_y, d_y_f32, (hipStream_t)stream);
}

// ---------------------------------------------------------------------------------------------
// operator level: tpu.A16MatMul
// ---------------------------------------------------------------------------------------------
int mi_a16mm_init(const mi_a16mm_attr *attr, mi_infer_param *p) {
  MI_REQUIRE(attr && p, MI_BAD_ARGUMENT, "mi_a16mm_init: null argument");
  p->handle = nullptr;
  MI_REQUIRE(p->inputs && p->n_inputs >= 4, MI_BAD_ARGUMENT, "mi_a16mm_init: expects input, weight, scale, zp[, bias]");
  const int dq = attr->dynamic_quant;
  MI_REQUIRE(dq == MI_DQ_NONE || dq == MI_DQ_INT || dq == MI_DQ_F8E4M3 || dq == MI_DQ_F4, MI_UNSUPPORTED,
             "mi_a16mm_init: dynamic_quant must be MI_DQ_NONE, MI_DQ_INT, MI_DQ_F8E4M3 or MI_DQ_F4");
  if (dq != MI_DQ_NONE) {
    MI_REQUIRE(attr->q_group_size != 0, MI_BAD_ARGUMENT,
               "mi_a16mm_init: dynamic quantization needs a group size (A16MatMul.cpp:42-43)");
    // A16MatMul.cpp:63-91 decodes F4 codes only from 4-bit and F8E4M3 codes only from 8-bit weights
    MI_REQUIRE((dq != MI_DQ_F8E4M3 || attr->weight_bits == 8) && (dq != MI_DQ_F4 || attr->weight_bits == 4),
               MI_UNSUPPORTED, "mi_a16mm_init: F8E4M3 needs 8-bit and F4 needs 4-bit weights");
    MI_REQUIRE(attr->q_group_size > 0 && attr->K % 128 == 0 &&
                   (attr->q_group_size == 32 || attr->q_group_size == 64 || attr->q_group_size % 128 == 0) &&
                   (dq != MI_DQ_INT || attr->weight_bits == 4 || attr->q_group_size <= 512),
               MI_UNSUPPORTED,
               "mi_a16mm_init: dynamic quantization is handled for K % 128 == 0 and groups of 32, 64 or k*128 (integer "
               "codes with 8-bit weights: up to 512, where the reference's f32 group product stops being exact)");
  }
  MI_REQUIRE(attr->weight_bits == 4 || attr->weight_bits == 8, MI_UNSUPPORTED, "mi_a16mm_init: weight_bits");
  MI_REQUIRE(attr->out_dtype == MI_DT_BF16 || attr->out_dtype == MI_DT_F16, MI_UNSUPPORTED, "mi_a16mm_init: out_dtype");
  const float *weight = p->inputs[1], *scale = p->inputs[2], *zp = p->inputs[3];
  const float *bias = p->n_inputs > 4 ? p->inputs[4] : nullptr;
  MI_REQUIRE(weight && scale && zp, MI_BAD_ARGUMENT, "mi_a16mm_init: weight, scale and zp must not be None");
  const int64_t K = attr->K, N = attr->N;
  MI_REQUIRE(K > 0 && N > 0, MI_BAD_ARGUMENT, "mi_a16mm_init: bad shape");
  if (!attr->w_transpose) {
    // A16MatMul.cpp:172-208 without the swap: weight stored [K, N/2], parameters per stored row k or per run of
    // q_group_size elements of the flattened [K, N] matrix; floats as the interpreter holds them, used as they are
    MI_REQUIRE(dq == MI_DQ_NONE, MI_UNSUPPORTED, "mi_a16mm_init: dynamic quantization needs w_transpose weights");
    MI_REQUIRE(N % 2 == 0, MI_UNSUPPORTED, "mi_a16mm_init: an untransposed 4-bit weight needs an even N");
    const int64_t nw = K * (N / 2);
    std::vector<uint8_t> wbytes((size_t)nw);
    for (int64_t i = 0; i < nw; ++i) {
      const float v = weight[i];
      MI_REQUIRE(v == truncf(v) && v >= 0.f && v <= 255.f, MI_UNSUPPORTED,
                 "mi_a16mm_init: weight is not a packed byte value");
      wbytes[(size_t)i] = (uint8_t)(int)v;
    }
    mi_a16_weight_desc d;
    d.K = K;
    d.N = N;
    d.weight_bits = attr->weight_bits;
    d.weight_signed = 0;
    d.q_group_size = attr->q_group_size;
    d.dtype = attr->out_dtype;
    d.chip = attr->chip;
    A16Handle *h = new (std::nothrow) A16Handle();
    MI_REQUIRE(h, MI_HIP_ERROR, "mi_a16mm_init: out of host memory");
    int rc = mi_a16_weight_create_kn(&h->w, &d, wbytes.data(), scale, zp, bias);
    if (rc == MI_SUCCESS) {
      hipError_t e = hipStreamCreateWithFlags(&h->stream, hipStreamNonBlocking);
      if (e != hipSuccess)
        rc = hip_fail(e, "hipStreamCreateWithFlags", __FILE__, __LINE__);
    }
    if (rc != MI_SUCCESS) {
      delete h;
      return rc;
    }
    p->handle = h;
    return MI_SUCCESS;
  }
  const int g = attr->q_group_size;
  MI_REQUIRE(g == 0 || (g > 0 && K % g == 0), MI_BAD_ARGUMENT, "mi_a16mm_init: K is not a multiple of q_group_size");
  MI_REQUIRE(K % 8 == 0, MI_UNSUPPORTED, "mi_a16mm_init: K must be a multiple of 8");
  const int64_t G = g ? K / g : 1;

  // float-expanded operands -> native storage
  const int64_t nw = attr->weight_bits == 4 ? N * (K / 2) : N * K;
  std::vector<uint8_t> wbytes((size_t)nw);
  bool neg = false;
  for (int64_t i = 0; i < nw; ++i) {
    float v = weight[i];
    MI_REQUIRE(v == truncf(v) && v >= -128.f && v <= 255.f, MI_UNSUPPORTED, "mi_a16mm_init: weight is not 8-bit integer valued");
    neg |= v < 0.f;
    wbytes[(size_t)i] = (uint8_t)(int)v;
  }
  MI_REQUIRE(!(neg && attr->weight_bits == 4), MI_UNSUPPORTED, "mi_a16mm_init: negative packed byte");
  if (neg)
    for (int64_t i = 0; i < nw; ++i)
      MI_REQUIRE(weight[i] <= 127.f, MI_UNSUPPORTED, "mi_a16mm_init: weight mixes int8 and uint8 ranges");
  std::vector<uint16_t> sbits((size_t)(N * G));
  std::vector<uint8_t> zbytes((size_t)(N * G));
  for (int64_t i = 0; i < N * G; ++i) {
    float s = scale[i];
    uint16_t b = attr->out_dtype == MI_DT_F16 ? h_f32_to_f16(s) : h_f32_to_bf16(s);
    float back = attr->out_dtype == MI_DT_F16 ? h_f16_to_f32(b) : h_bf16_to_f32(b);
    MI_REQUIRE(back == s, MI_UNSUPPORTED, "mi_a16mm_init: scale is not representable in the 16-bit activation type");
    sbits[(size_t)i] = b;
    float z = zp[i];
    MI_REQUIRE(z == truncf(z) && z >= 0.f && z <= 255.f, MI_UNSUPPORTED, "mi_a16mm_init: zero point is not a u8 value");
    zbytes[(size_t)i] = (uint8_t)(int)z;
  }
  mi_a16_weight_desc d;
  d.K = K;
  d.N = N;
  d.weight_bits = attr->weight_bits;
  d.weight_signed = neg ? 1 : 0;
  d.q_group_size = g;
  d.dtype = attr->out_dtype;
  d.chip = attr->chip;
  A16Handle *h = new (std::nothrow) A16Handle();
  MI_REQUIRE(h, MI_HIP_ERROR, "mi_a16mm_init: out of host memory");
  int rc = mi_a16_weight_create(&h->w, &d, wbytes.data(), sbits.data(), zbytes.data(), bias);
  if (rc == MI_SUCCESS) {
    hipError_t e = hipStreamCreateWithFlags(&h->stream, hipStreamNonBlocking);
    if (e != hipSuccess)
      rc = hip_fail(e, "hipStreamCreateWithFlags", __FILE__, __LINE__);
  }
  if (rc != MI_SUCCESS) {
    delete h;
    return rc;
  }
  p->handle = h;
  return MI_SUCCESS;
}

int mi_a16mm_inference(const mi_a16mm_attr *attr, mi_infer_param *p) {
  MI_REQUIRE(attr && p, MI_BAD_ARGUMENT, "mi_a16mm_inference: null argument");
  MI_REQUIRE(p->handle, MI_BAD_ARGUMENT, "mi_a16mm_inference: init has not been called");
  A16Handle *h = (A16Handle *)p->handle;
  MI_REQUIRE(h->magic == 0xA16A16u, MI_BAD_ARGUMENT, "mi_a16mm_inference: handle does not belong to an A16MatMul");
  MI_REQUIRE(p->inputs && p->n_inputs >= 1 && p->inputs[0] && p->outputs && p->n_outputs >= 1 && p->outputs[0],
             MI_BAD_ARGUMENT, "mi_a16mm_inference: null input or output");
  MI_REQUIRE(attr->K == h->w->K && attr->N == h->w->N, MI_BAD_ARGUMENT, "mi_a16mm_inference: K/N differ from init");
  const int64_t M = attr->M, K = attr->K, N = attr->N;
  MI_REQUIRE(M >= 0, MI_BAD_ARGUMENT, "mi_a16mm_inference: negative M");
  if (M == 0)
    return MI_SUCCESS;
  const int64_t nx = M * K, ny = M * N;
  const bool small_in = nx <= SMALL_CALL_ELEMS, small_out = ny <= SMALL_CALL_ELEMS;
  const int f16 = h->w->dtype == MI_DT_F16;
  int rc;
  if ((rc = h->d_x.reserve((size_t)nx * 2)))
    return rc;
  const float *src;
  if (small_in) {
    if ((rc = h->h_x.reserve((size_t)nx * 4)))
      return rc;
    memcpy(h->h_x.ptr, p->inputs[0], (size_t)nx * 4);
    src = (const float *)h->h_x.ptr;
  } else {
    if ((rc = h->d_xf.reserve((size_t)nx * 4)))
      return rc;
    MI_HIP(hipMemcpyAsync(h->d_xf.ptr, p->inputs[0], (size_t)nx * 4, hipMemcpyHostToDevice, h->stream));
    src = (const float *)h->d_xf.ptr;
  }
  stage_f32_to_16_kernel<<<dim3(stage_grid(nx)), dim3(256), 0, h->stream>>>(src, (uint16_t *)h->d_x.ptr, nx, f16);
  if ((rc = small_out ? h->h_y.reserve((size_t)ny * 2) : h->d_y.reserve((size_t)ny * 2)))
    return rc;
  uint16_t *y16 = (uint16_t *)(small_out ? h->h_y.ptr : h->d_y.ptr);
  if (attr->dynamic_quant != MI_DQ_NONE)
    rc = a16_dq_launch(h->w, attr->dynamic_quant, (const uint16_t *)h->d_x.ptr, M, y16, nullptr, h->stream);
  else
    rc = a16_launch(h->w, (const uint16_t *)h->d_x.ptr, M, y16, nullptr, h->stream);
  if (rc != MI_SUCCESS)
    return rc;
  float *y = p->outputs[0];
  if (small_out) {
    MI_HIP(hipStreamSynchronize(h->stream));
    for (int64_t i = 0; i < ny; ++i)
      y[i] = f16 ? h_f16_to_f32(y16[i]) : h_bf16_to_f32(y16[i]);
  } else {
    if ((rc = h->d_yf.reserve((size_t)ny * 4)))
      return rc;
    expand_16_to_f32_kernel<<<dim3(stage_grid(ny)), dim3(256), 0, h->stream>>>(y16, (float *)h->d_yf.ptr, ny, f16);
    MI_HIP(hipMemcpyAsync(y, h->d_yf.ptr, (size_t)ny * 4, hipMemcpyDeviceToHost, h->stream));
    MI_HIP(hipStreamSynchronize(h->stream));
  }
  return MI_SUCCESS;
}

void mi_a16mm_deinit(mi_infer_param *p) {
  if (!p || !p->handle)
    return;
  A16Handle *h = (A16Handle *)p->handle;
  if (h->magic == 0xA16A16u)
    delete h;
  p->handle = nullptr;
}

// ---------------------------------------------------------------------------------------------
// device level: int8 matmul / requant
// ---------------------------------------------------------------------------------------------
int mi_i8mm_launch(const void *d_a, int a_unsigned, const void *d_b, int b_unsigned, int right_transpose,
                   const int32_t *d_bias, int64_t M, int64_t K, int64_t N, int64_t input_zp, int64_t right_zp,
                   int do_relu, int64_t relu_limit, const mi_requant_desc *rq, void *d_out, int32_t *d_acc,
                   void *stream) {
  return i8mm_launch(d_a, a_unsigned, d_b, b_unsigned, right_transpose, d_bias, M, K, N, input_zp, right_zp, do_relu,
                     relu_limit, rq, d_out, d_acc, (hipStream_t)stream);
}

int mi_requant_launch(const int32_t *d_in, void *d_out, int64_t outer, int64_t channels, int64_t inner,
                      int64_t input_zp, const mi_requant_desc *rq, void *stream) {
  return requant_launch(d_in, d_out, outer, channels, inner, input_zp, rq, (hipStream_t)stream);
}

}  // extern "C"

// ---------------------------------------------------------------------------------------------
// operator level: tpu.MatMul (quantized)
// ---------------------------------------------------------------------------------------------
namespace mi {

struct I8Handle {
  uint32_t magic = 0x18181818u;
  int64_t K = 0, N = 0;
  bool right_cached = false;
  bool right_pre_transposed = false;  // a [K, N] weight is kept as [N, K]
  int right_unsigned = 0;
  DevBuf d_a, d_b, d_bias, d_multi, d_out;
  Pinned h_a, h_b, h_out;
  bool has_bias = false, has_multi = false;
  hipStream_t stream = nullptr;
  ~I8Handle() {
    if (stream) {
      release_stream_workspaces(stream);
      (void)hipStreamDestroy(stream);
    }
  }
};

static int out_elem_size(int dt) {
  switch (dt) {
  case MI_DT_I8:
  case MI_DT_U8:
    return 1;
  case MI_DT_I16:
  case MI_DT_U16:
    return 2;
  default:
    return 4;
  }
}

// float-expanded 8-bit integers -> bytes; reports whether they are int8 or uint8 valued.  A call of the operator spends
// its time here and in the expansion of the result, not on the GPU, so the loop is written with SSE2 intrinsics (every
// x86-64 host has them; left to the auto-vectorizer the same loop came out scalar in this translation unit, five times
// slower).  Per element: truncate to int and convert back (stands in for truncf; NaN compares unequal), check the
// range on the integer, take the low byte.  Bytes past the last multiple of 16 go through the scalar form.
#if defined(__SSE2__)
// The same loop eight floats at a time where the host has AVX2 (checked once at run time; the translation unit is not
// compiled for it): 32 values per pass, bytes put back in order after the two in-lane packs.  Returns the number of
// values done (a multiple of 32); the flags are ORed into.
__attribute__((target("avx2"))) static int64_t floats_to_bytes_avx2(const float *src, int64_t n, uint8_t *dst, int *bad,
                                                                    int *any_neg, int *any_big) {
  __m256i vbad = _mm256_setzero_si256(), vneg = _mm256_setzero_si256(), vbig = _mm256_setzero_si256();
  const __m256i c128 = _mm256_set1_epi32(128), c383 = _mm256_set1_epi32(383 - 0x7fffffff - 1);
  const __m256i sign = _mm256_set1_epi32(-0x7fffffff - 1), c127 = _mm256_set1_epi32(127), lowbyte = _mm256_set1_epi32(0xff);
  const __m256i order = _mm256_setr_epi32(0, 4, 1, 5, 2, 6, 3, 7);
  int64_t i = 0;
  for (; i + 32 <= n; i += 32) {
    __m256i q[4];
    for (int u = 0; u < 4; ++u) {
      const __m256 v = _mm256_loadu_ps(src + i + 8 * u);
      const __m256i iv = _mm256_cvttps_epi32(v);
      vbad = _mm256_or_si256(vbad, _mm256_castps_si256(_mm256_cmp_ps(_mm256_cvtepi32_ps(iv), v, _CMP_NEQ_UQ)));
      vbad = _mm256_or_si256(vbad, _mm256_cmpgt_epi32(_mm256_xor_si256(_mm256_add_epi32(iv, c128), sign), c383));
      vneg = _mm256_or_si256(vneg, iv);
      vbig = _mm256_or_si256(vbig, _mm256_sub_epi32(c127, iv));
      q[u] = _mm256_and_si256(iv, lowbyte);
    }
    const __m256i packed = _mm256_packus_epi16(_mm256_packs_epi32(q[0], q[1]), _mm256_packs_epi32(q[2], q[3]));
    _mm256_storeu_si256((__m256i *)(dst + i), _mm256_permutevar8x32_epi32(packed, order));
  }
  *bad |= _mm256_movemask_epi8(vbad) != 0;
  *any_neg |= _mm256_movemask_ps(_mm256_castsi256_ps(vneg)) != 0;
  *any_big |= _mm256_movemask_ps(_mm256_castsi256_ps(vbig)) != 0;
  return i;
}
__attribute__((target("avx2"))) static int64_t i8_to_floats_avx2(const int8_t *src, int64_t n, float *y, bool is_unsigned) {
  int64_t i = 0;
  for (; i + 16 <= n; i += 16) {
    const __m128i b = _mm_loadu_si128((const __m128i *)(src + i));
    const __m128i hi = _mm_unpackhi_epi64(b, b);
    const __m256i lo32 = is_unsigned ? _mm256_cvtepu8_epi32(b) : _mm256_cvtepi8_epi32(b);
    const __m256i hi32 = is_unsigned ? _mm256_cvtepu8_epi32(hi) : _mm256_cvtepi8_epi32(hi);
    _mm256_storeu_ps(y + i, _mm256_cvtepi32_ps(lo32));
    _mm256_storeu_ps(y + i + 8, _mm256_cvtepi32_ps(hi32));
  }
  return i;
}
static bool host_has_avx2() {
  static const bool yes = __builtin_cpu_supports("avx2");
  return yes;
}
#endif

static int floats_to_bytes(const float *src, int64_t n, uint8_t *dst, int *is_unsigned, const char *who) {
  int bad = 0, any_neg = 0, any_big = 0;
  int64_t i = 0;
#if defined(__SSE2__)
  if (host_has_avx2())
    i = floats_to_bytes_avx2(src, n, dst, &bad, &any_neg, &any_big);
  __m128i vbad = _mm_setzero_si128(), vneg = _mm_setzero_si128(), vbig = _mm_setzero_si128();
  const __m128i c128 = _mm_set1_epi32(128), c383 = _mm_set1_epi32(383 - 0x7fffffff - 1), sign = _mm_set1_epi32(-0x7fffffff - 1);
  const __m128i c127 = _mm_set1_epi32(127), lowbyte = _mm_set1_epi32(0xff);
  for (; i + 16 <= n; i += 16) {
    __m128i q[4];
    for (int u = 0; u < 4; ++u) {
      const __m128 v = _mm_loadu_ps(src + i + 4 * u);
      const __m128i iv = _mm_cvttps_epi32(v);  // out of range and NaN give INT_MIN, caught by the range check
      vbad = _mm_or_si128(vbad, _mm_castps_si128(_mm_cmpneq_ps(_mm_cvtepi32_ps(iv), v)));
      // unsigned (iv + 128) > 383, as a signed compare on both sides flipped
      vbad = _mm_or_si128(vbad, _mm_cmpgt_epi32(_mm_xor_si128(_mm_add_epi32(iv, c128), sign), c383));
      vneg = _mm_or_si128(vneg, iv);                        // sign bit: some value below zero
      vbig = _mm_or_si128(vbig, _mm_sub_epi32(c127, iv));   // sign bit: some value above 127
      q[u] = _mm_and_si128(iv, lowbyte);
    }
    _mm_storeu_si128((__m128i *)(dst + i), _mm_packus_epi16(_mm_packs_epi32(q[0], q[1]), _mm_packs_epi32(q[2], q[3])));
  }
  bad |= _mm_movemask_epi8(vbad) != 0;
  any_neg |= (_mm_movemask_ps(_mm_castsi128_ps(vneg)) != 0);
  any_big |= (_mm_movemask_ps(_mm_castsi128_ps(vbig)) != 0);
#endif
  for (; i < n; ++i) {
    const float v = src[i];
    const bool in_range = v >= -128.f && v <= 255.f;  // false for NaN
    const int32_t iv = in_range ? (int32_t)v : 0;
    bad |= !in_range || (float)iv != v;
    any_neg |= iv < 0;
    any_big |= iv > 127;
    dst[i] = (uint8_t)iv;
  }
  MI_REQUIRE(!bad && !(any_neg && any_big), MI_UNSUPPORTED,
             std::string(who) + ": operand does not hold the values of one 8-bit integer type");
  *is_unsigned = any_big;
  return MI_SUCCESS;
}

static int floats_to_i32_dev(const float *src, int64_t n, DevBuf &buf, hipStream_t st) {
  std::vector<int32_t> tmp((size_t)n);
  for (int64_t i = 0; i < n; ++i)
    tmp[(size_t)i] = (int32_t)(int64_t)src[i];
  int rc = buf.reserve((size_t)n * 4);
  if (rc)
    return rc;
  MI_HIP(hipMemcpyAsync(buf.ptr, tmp.data(), (size_t)n * 4, hipMemcpyHostToDevice, st));
  MI_HIP(hipStreamSynchronize(st));
  return MI_SUCCESS;
}

static int upload_right(I8Handle *h, const mi_i8mm_attr *attr, const float *right) {
  const int64_t n = attr->K * attr->N;
  int rc = h->h_b.reserve((size_t)n);
  if (rc)
    return rc;
  if ((rc = floats_to_bytes(right, n, (uint8_t *)h->h_b.ptr, &h->right_unsigned, "mi_i8mm")))
    return rc;
  if ((rc = h->d_b.reserve((size_t)n)))
    return rc;
  h->right_pre_transposed = false;
  if (attr->right_is_weight && !attr->right_transpose) {
    // a [K, N] weight is laid out [N, K] once, here, instead of on every call (the kernels read both operands along K)
    DevBuf tmp;
    if ((rc = tmp.reserve((size_t)n)))
      return rc;
    MI_HIP(hipMemcpyAsync(tmp.ptr, h->h_b.ptr, (size_t)n, hipMemcpyHostToDevice, h->stream));
    if ((rc = permute_launch(tmp.ptr, h->d_b.ptr, 1, 0, 1, 1, attr->K, attr->N, h->stream)))
      return rc;
    MI_HIP(hipStreamSynchronize(h->stream));  // tmp is freed on return
    h->right_pre_transposed = true;
    return MI_SUCCESS;
  }
  MI_HIP(hipMemcpyAsync(h->d_b.ptr, h->h_b.ptr, (size_t)n, hipMemcpyHostToDevice, h->stream));
  return MI_SUCCESS;
}

static int check_i8_attr(const mi_i8mm_attr *a, const char *who) {
  MI_REQUIRE(a->M >= 0 && a->K > 0 && a->N > 0, MI_BAD_ARGUMENT, std::string(who) + ": bad shape");
  const int o = a->out_dtype;
  MI_REQUIRE(o == MI_DT_I8 || o == MI_DT_U8 || o == MI_DT_I16 || o == MI_DT_U16 || o == MI_DT_I32, MI_UNSUPPORTED,
             std::string(who) + ": output type not handled");
  if (o != MI_DT_I32) {
    const int q = a->quant_mode;
    if (a->chip == MI_CHIP_CV18XX)
      MI_REQUIRE(q == MI_RQ_MULTIPLIER_SHIFT || q == MI_RQ_ONLY_SHIFT || q == MI_RQ_QDM || q == MI_RQ_TFLITE ||
                     q == MI_RQ_TFLITE_LSHIFT,
                 MI_UNSUPPORTED, std::string(who) + ": requant mode not handled");
    else
      MI_REQUIRE(q == MI_RQ_MULTIPLIER_SHIFT || q == MI_RQ_TFLITE || q == MI_RQ_TFLITE_LSHIFT || q == MI_RQ_ONLY_SCALE,
                 MI_UNSUPPORTED, std::string(who) + ": requant mode not handled");
    // the reference asserts on the per-channel flavour of OnlyScale (MatMul.cpp:674-676)
    MI_REQUIRE(!(q == MI_RQ_ONLY_SCALE && a->fuse_rq), MI_UNSUPPORTED,
               std::string(who) + ": OnlyScale with fuse_rq is not supported; use MultiplierShift");
    if (q == MI_RQ_ONLY_SCALE)
      return MI_SUCCESS;
    MI_REQUIRE(a->multipliers && a->n_multipliers >= 1 && a->rshifts && a->n_rshifts >= 1, MI_BAD_ARGUMENT,
               std::string(who) + ": multipliers / rshifts missing");
  }
  return MI_SUCCESS;
}

// The scalar part of the requantization of tpu::MatMulOp::inference (MatMul.cpp:636-727) as a device descriptor; the
// caller adds per-channel / per-batch arrays.
static void fill_i8_rq(const mi_i8mm_attr *attr, mi_requant_desc *rq) {
  memset(rq, 0, sizeof(*rq));
  rq->chip = attr->chip;
  rq->out_dtype = attr->out_dtype;
  rq->quant_mode = attr->quant_mode;
  rq->multiplier = attr->multipliers && attr->n_multipliers > 0 ? (int32_t)attr->multipliers[0] : 1;
  rq->shift = attr->rshifts && attr->n_rshifts > 0 ? (int32_t)attr->rshifts[0] : 0;
  if (attr->chip == MI_CHIP_CV18XX) {
    // MatMul.cpp:638-664: per-batch multiplier/rshift, half away from zero, no zero point
    rq->round_mode = MI_ROUND_HALF_AWAY_FROM_ZERO;
    rq->zp = 0;
  } else if (attr->quant_mode == MI_RQ_ONLY_SCALE) {
    // MatMul.cpp:683-691: (int32)roundf(acc * (float)out_scales[0]) + zero point
    rq->round_mode = MI_ROUND_HALF_AWAY_FROM_ZERO;
    rq->zp = (int32_t)attr->out_zp;
    rq->only_scale = (float)attr->out_scale;
  } else if (attr->quant_mode == MI_RQ_MULTIPLIER_SHIFT) {
    // MatMul.cpp:708-726: default rounding of applyMultiplierAndRShift is half up (MathUtils.h:178-181)
    rq->round_mode = MI_ROUND_HALF_UP;
    rq->zp = (int32_t)attr->out_zp;
  } else {
    // MatMul.cpp:696-707: MultiplyByQuantizedMultiplier(acc, mult, -rshift), half away from zero
    rq->round_mode = MI_ROUND_HALF_AWAY_FROM_ZERO;
    rq->zp = (int32_t)attr->out_zp;
  }
}

static void bytes_to_floats(const void *ho, int out_dtype, int64_t n, float *y) {
  int64_t i0 = 0;
#if defined(__SSE2__)
  if ((out_dtype == MI_DT_I8 || out_dtype == MI_DT_U8) && host_has_avx2())
    i0 = i8_to_floats_avx2((const int8_t *)ho, n, y, out_dtype == MI_DT_U8);
#endif
  switch (out_dtype) {
  case MI_DT_I8:
    for (int64_t i = i0; i < n; ++i) y[i] = (float)((const int8_t *)ho)[i];
    break;
  case MI_DT_U8:
    for (int64_t i = i0; i < n; ++i) y[i] = (float)((const uint8_t *)ho)[i];
    break;
  case MI_DT_I16:
    for (int64_t i = 0; i < n; ++i) y[i] = (float)((const int16_t *)ho)[i];
    break;
  case MI_DT_U16:
    for (int64_t i = 0; i < n; ++i) y[i] = (float)((const uint16_t *)ho)[i];
    break;
  default:
    for (int64_t i = 0; i < n; ++i) y[i] = (float)((const int32_t *)ho)[i];
    break;
  }
}

}  // namespace mi

extern "C" {

int mi_i8mm_init(const mi_i8mm_attr *attr, mi_infer_param *p) {
  MI_REQUIRE(attr && p, MI_BAD_ARGUMENT, "mi_i8mm_init: null argument");
  p->handle = nullptr;
  MI_REQUIRE(p->inputs && p->n_inputs >= 2 && p->inputs[0] && p->inputs[1], MI_BAD_ARGUMENT,
             "mi_i8mm_init: input and right must not be None");
  int rc = check_i8_attr(attr, "mi_i8mm_init");
  if (rc)
    return rc;
  MI_REQUIRE(mi_device_count() > 0, MI_HIP_ERROR, "mi_i8mm_init: no GPU visible");
  I8Handle *h = new (std::nothrow) I8Handle();
  MI_REQUIRE(h, MI_HIP_ERROR, "mi_i8mm_init: out of host memory");
  h->K = attr->K;
  h->N = attr->N;
  hipError_t e = hipStreamCreateWithFlags(&h->stream, hipStreamNonBlocking);
  if (e != hipSuccess) {
    delete h;
    return hip_fail(e, "hipStreamCreateWithFlags", __FILE__, __LINE__);
  }
  const float *bias = p->n_inputs > 2 ? p->inputs[2] : nullptr;
  const float *multi = p->n_inputs > 3 ? p->inputs[3] : nullptr;
  if (attr->right_is_weight) {
    rc = upload_right(h, attr, p->inputs[1]);
    h->right_cached = rc == MI_SUCCESS;
  }
  if (rc == MI_SUCCESS && bias) {
    rc = floats_to_i32_dev(bias, attr->N, h->d_bias, h->stream);
    h->has_bias = rc == MI_SUCCESS && attr->right_is_weight;  // constant only beside a weight; else re-read per call
  }
  if (rc == MI_SUCCESS && multi && attr->fuse_rq) {
    rc = floats_to_i32_dev(multi, attr->N, h->d_multi, h->stream);
    h->has_multi = rc == MI_SUCCESS && attr->right_is_weight;
  }
  if (rc == MI_SUCCESS) {
    e = hipStreamSynchronize(h->stream);
    if (e != hipSuccess)
      rc = hip_fail(e, "hipStreamSynchronize", __FILE__, __LINE__);
  }
  if (rc != MI_SUCCESS) {
    delete h;
    return rc;
  }
  p->handle = h;
  return MI_SUCCESS;
}

int mi_i8mm_inference(const mi_i8mm_attr *attr, mi_infer_param *p) {
  MI_REQUIRE(attr && p, MI_BAD_ARGUMENT, "mi_i8mm_inference: null argument");
  if (!p->handle) {  // the reference initialises lazily (MatMul.cpp:441-443)
    int rc0 = mi_i8mm_init(attr, p);
    if (rc0)
      return rc0;
  }
  I8Handle *h = (I8Handle *)p->handle;
  MI_REQUIRE(h->magic == 0x18181818u, MI_BAD_ARGUMENT, "mi_i8mm_inference: handle does not belong to a MatMul");
  MI_REQUIRE(p->inputs && p->n_inputs >= 2 && p->inputs[0] && p->inputs[1] && p->outputs && p->n_outputs >= 1 &&
                 p->outputs[0],
             MI_BAD_ARGUMENT, "mi_i8mm_inference: null input or output");
  int rc = check_i8_attr(attr, "mi_i8mm_inference");
  if (rc)
    return rc;
  MI_REQUIRE(attr->K == h->K && attr->N == h->N, MI_BAD_ARGUMENT, "mi_i8mm_inference: K/N differ from init");
  const int64_t M = attr->M, K = attr->K, N = attr->N;
  if (M == 0)
    return MI_SUCCESS;
  const int osz = out_elem_size(attr->out_dtype);
  if ((rc = h->h_a.reserve((size_t)M * K)) || (rc = h->d_a.reserve((size_t)M * K)) ||
      (rc = h->h_out.reserve((size_t)M * N * osz)) || (rc = h->d_out.reserve((size_t)M * N * osz)))
    return rc;
  int a_unsigned = 0;
  if ((rc = floats_to_bytes(p->inputs[0], M * K, (uint8_t *)h->h_a.ptr, &a_unsigned, "mi_i8mm_inference")))
    return rc;
  if ((size_t)M * K <= SMALL_I8_CALL_BYTES && ((size_t)M * K) % 16 == 0)  // read over the bus by a kernel: no copy command
    copy16_kernel<<<dim3(stage_grid(M * K / 16)), dim3(256), 0, h->stream>>>((const uint4 *)h->h_a.ptr,
                                                                              (uint4 *)h->d_a.ptr, M * K / 16);
  else
    MI_HIP(hipMemcpyAsync(h->d_a.ptr, h->h_a.ptr, (size_t)M * K, hipMemcpyHostToDevice, h->stream));
  if (!h->right_cached && (rc = upload_right(h, attr, p->inputs[1])))
    return rc;
  const float *bias = p->n_inputs > 2 ? p->inputs[2] : nullptr;
  const float *multi = p->n_inputs > 3 ? p->inputs[3] : nullptr;
  if (bias && !h->has_bias) {
    if ((rc = floats_to_i32_dev(bias, N, h->d_bias, h->stream)))
      return rc;
    h->has_bias = attr->right_is_weight;  // weights' bias is constant; otherwise re-upload each call
  }
  mi_requant_desc rq;
  const mi_requant_desc *rqp = nullptr;
  if (attr->out_dtype != MI_DT_I32) {
    rqp = &rq;
    fill_i8_rq(attr, &rq);
    if (attr->chip != MI_CHIP_CV18XX && attr->quant_mode == MI_RQ_MULTIPLIER_SHIFT && attr->fuse_rq) {
      MI_REQUIRE(multi, MI_BAD_ARGUMENT, "mi_i8mm_inference: fuse_rq needs the multi operand");
      if (!h->has_multi) {
        if ((rc = floats_to_i32_dev(multi, N, h->d_multi, h->stream)))
          return rc;
        h->has_multi = attr->right_is_weight;
      }
      rq.d_multiplier = (const int32_t *)h->d_multi.ptr;
    }
  }
  const int64_t relu_limit = attr->relu_limit > 0.0 ? (int64_t)floor(attr->relu_limit) : -1;
  // a small result goes to the pinned host buffer through a copy kernel's 16-byte stores over the bus (no copy command;
  // the matmul's own epilogue may store single bytes, which the bus takes one at a time)
  const bool out_direct = false;
  const bool out_by_kernel = (size_t)M * N * osz <= SMALL_I8_CALL_BYTES && ((size_t)M * N * osz) % 16 == 0;
  rc = i8mm_launch(h->d_a.ptr, a_unsigned, h->d_b.ptr, h->right_unsigned, attr->right_transpose || h->right_pre_transposed,
                   bias ? (const int32_t *)h->d_bias.ptr : nullptr, M, K, N, attr->input_zp, attr->right_zp,
                   attr->do_relu, relu_limit, rqp, out_direct ? h->h_out.ptr : h->d_out.ptr, nullptr, h->stream);
  if (rc)
    return rc;
  if (out_by_kernel)
    copy16_kernel<<<dim3(stage_grid(M * N * osz / 16)), dim3(256), 0, h->stream>>>((const uint4 *)h->d_out.ptr,
                                                                                 (uint4 *)h->h_out.ptr, M * N * osz / 16);
  else
    MI_HIP(hipMemcpyAsync(h->h_out.ptr, h->d_out.ptr, (size_t)M * N * osz, hipMemcpyDeviceToHost, h->stream));
  MI_HIP(hipStreamSynchronize(h->stream));
  bytes_to_floats(h->h_out.ptr, attr->out_dtype, M * N, p->outputs[0]);
  return MI_SUCCESS;
}

// one operator handle per batch (each caches its own right operand when that is a weight)
struct I8BatchHandle {
  uint32_t magic = 0x18B18B18u;
  std::vector<void *> per_batch;
};

// a MatMul whose operands or output MatMul::run transposes: everything in one handle, nothing cached between calls
// (these are matmuls of two activations)
struct I8NdHandle {
  uint32_t magic = 0x18D18D18u;
  mi::DevBuf d_a, d_a2, d_b, d_b2, d_acc, d_acc2, d_out, d_bias, d_multi, d_mult_b, d_rs_b;
  mi::Pinned h_a, h_b, h_out;
  hipStream_t stream = nullptr;
  ~I8NdHandle() {
    if (stream) {
      mi::release_stream_workspaces(stream);
      (void)hipStreamDestroy(stream);
    }
  }
};

void mi_i8mm_deinit(mi_infer_param *p) {
  if (!p || !p->handle)
    return;
  I8Handle *h = (I8Handle *)p->handle;
  if (h->magic == 0x18181818u) {
    delete h;
  } else if (h->magic == 0x18D18D18u) {
    delete (I8NdHandle *)p->handle;
  } else if (h->magic == 0x18B18B18u) {
    I8BatchHandle *bh = (I8BatchHandle *)p->handle;
    for (void *one : bh->per_batch)
      if (one && ((I8Handle *)one)->magic == 0x18181818u)
        delete (I8Handle *)one;
    delete bh;
  }
  p->handle = nullptr;
}

int mi_matmul_parse_param(const mi_matmul_shapes *sh, int right_transpose, int chip, mi_matmul_param *out) {
  MI_REQUIRE(sh && out, MI_BAD_ARGUMENT, "mi_matmul_parse_param: null argument");
  MI_REQUIRE(sh->a_dims >= 1 && sh->a_dims <= 8 && sh->b_dims >= 1 && sh->b_dims <= 8 && sh->o_dims >= 0 && sh->o_dims <= 8,
             MI_BAD_ARGUMENT, "mi_matmul_parse_param: ranks must be 1 .. 8");
  std::vector<int64_t> a(sh->a_shape, sh->a_shape + sh->a_dims), b(sh->b_shape, sh->b_shape + sh->b_dims),
      o(sh->o_shape, sh->o_shape + sh->o_dims);
  mi_matmul_param p;
  memset(&p, 0, sizeof(p));
  p.right_transpose = right_transpose;
  p.left_transpose = sh->left_transpose;
  p.output_transpose = sh->output_transpose;
  p.hdim_is_batch = sh->hdim_is_batch;
  p.batch = p.batch_low = 1;
  if (b.size() == 1) {  // a vector on the right is a one-column matrix (MatMul.cpp:44-50)
    MI_REQUIRE(!right_transpose, MI_BAD_ARGUMENT, "mi_matmul_parse_param: 1-D right operand with right_transpose");
    b.push_back(1);
    o.push_back(1);
  }
  if (a.size() == 1) {  // a vector on the left is a one-row matrix (:51-57)
    MI_REQUIRE(!sh->left_transpose, MI_BAD_ARGUMENT, "mi_matmul_parse_param: 1-D left operand with left_transpose");
    a.insert(a.begin(), 1);
    o.insert(o.begin(), 1);
  }
  const size_t ad = a.size(), bd = b.size(), od = o.size();
  MI_REQUIRE(od >= 2 && (!p.hdim_is_batch || (ad >= 3 && bd >= 3 && od >= 3)), MI_BAD_ARGUMENT,
             "mi_matmul_parse_param: output rank too small for these operands");
  const bool bm1684x = chip == MI_CHIP_BM168X;
  if (right_transpose && p.hdim_is_batch) {  // :63-72
    p.K = bm1684x ? b[bd - 1] : b[bd - 3];
    p.N = bm1684x ? b[bd - 3] : b[bd - 1];
  } else {
    p.N = right_transpose ? b[bd - 2] : b[bd - 1];
    p.K = right_transpose ? b[bd - 1] : b[bd - 2];
  }
  p.M = sh->left_transpose ? (p.hdim_is_batch ? a[ad - 3] : a[ad - 1]) : a[ad - 2];  // :81-90
  for (size_t i = 0; i + 2 < od; ++i)
    p.batch *= o[i];
  if (p.hdim_is_batch) {  // :96-104
    p.batch = o[0];
    if (!sh->output_transpose && chip == MI_CHIP_CV18XX) {
      p.batch_low = o[1];
    } else {
      p.batch_low = o[2];
      p.output_transpose = 1;
    }
  } else {  // :105-133
    int64_t right_batch = 1;
    for (size_t i = 0; i + 2 < bd; ++i)
      right_batch *= b[i];
    if (right_batch != p.batch && right_batch == 1)
      p.batch = 1;  // a right operand without batch dims: the left batch dims become rows
    if (p.batch > 1 || od <= 2) {
      p.M = sh->output_transpose ? o[od - 1] : o[od - 2];
    } else {
      p.M = 1;
      for (size_t i = 0; i + 1 < od; ++i)
        p.M *= o[i];
    }
    int64_t b_inner = 1;
    for (size_t i = 1; i + 2 < bd; ++i)
      b_inner *= b[i];
    if (a[0] == b[0] && b_inner == 1 && bd > 2) {
      p.batch = b[0];
      int64_t a_inner = 1;
      for (size_t i = 1; i + 2 < ad; ++i)
        a_inner *= a[i];
      const size_t idx = od - 2 + (sh->left_transpose ? 1 : 0);
      MI_REQUIRE(idx < ad, MI_BAD_ARGUMENT, "mi_matmul_parse_param: left rank too small for the output");
      p.M = a[idx] * a_inner;
    }
  }
  *out = p;
  return MI_SUCCESS;
}

// tpu.MatMul with left_transpose, output_transpose or hdim_is_batch: the operands are re-laid on the device as
// MatMul::run does on the host (lib/Support/Dnnl/MatMul.cpp:167-201), every batch's product leaves as int32
// accumulators, the output is re-laid (:228-238) and requantized in one pass over the flat result, per-channel operands
// indexed by the output's last dimension (MatMul.cpp:666-668).
static int i8mm_inference_relaid(const mi_i8mm_attr *attr, const mi_matmul_shapes *shapes, const mi_matmul_param &mp,
                                 mi_infer_param *p) {
  const int64_t B = mp.batch, BL = mp.batch_low, FB = B * BL, M = mp.M, K = mp.K, N = mp.N;
  const int64_t a_num = FB * M * K, b_num = FB * K * N, o_num = FB * M * N;
  MI_REQUIRE(shapes->o_dims >= 1, MI_BAD_ARGUMENT, "mi_i8mm_inference_nd: output shape missing");
  const int64_t n_last = shapes->o_shape[shapes->o_dims - 1];
  I8NdHandle *h = (I8NdHandle *)p->handle;
  if (!h) {
    MI_REQUIRE(mi_device_count() > 0, MI_HIP_ERROR, "mi_i8mm_inference_nd: no GPU visible");
    h = new (std::nothrow) I8NdHandle();
    MI_REQUIRE(h, MI_HIP_ERROR, "mi_i8mm_inference_nd: out of host memory");
    hipError_t e = hipStreamCreateWithFlags(&h->stream, hipStreamNonBlocking);
    if (e != hipSuccess) {
      delete h;
      return hip_fail(e, "hipStreamCreateWithFlags", __FILE__, __LINE__);
    }
    p->handle = h;
  }
  MI_REQUIRE(h->magic == 0x18D18D18u, MI_BAD_ARGUMENT, "mi_i8mm_inference_nd: the handle belongs to another op");
  if (o_num == 0)
    return MI_SUCCESS;
  const int osz = out_elem_size(attr->out_dtype);
  int rc;
  if ((rc = h->h_a.reserve((size_t)a_num)) || (rc = h->d_a.reserve((size_t)a_num)) ||
      (rc = h->h_b.reserve((size_t)b_num)) || (rc = h->d_b.reserve((size_t)b_num)) ||
      (rc = h->d_acc.reserve((size_t)o_num * 4)) || (rc = h->h_out.reserve((size_t)o_num * 4)) ||
      (rc = h->d_out.reserve((size_t)o_num * osz)))
    return rc;
  int a_unsigned = 0, b_unsigned = 0;
  if ((rc = floats_to_bytes(p->inputs[0], a_num, (uint8_t *)h->h_a.ptr, &a_unsigned, "mi_i8mm_inference_nd")) ||
      (rc = floats_to_bytes(p->inputs[1], b_num, (uint8_t *)h->h_b.ptr, &b_unsigned, "mi_i8mm_inference_nd")))
    return rc;
  MI_HIP(hipMemcpyAsync(h->d_a.ptr, h->h_a.ptr, (size_t)a_num, hipMemcpyHostToDevice, h->stream));
  MI_HIP(hipMemcpyAsync(h->d_b.ptr, h->h_b.ptr, (size_t)b_num, hipMemcpyHostToDevice, h->stream));
  const uint8_t *pa = (const uint8_t *)h->d_a.ptr, *pb = (const uint8_t *)h->d_b.ptr;
  if (mp.left_transpose) {
    if ((rc = h->d_a2.reserve((size_t)a_num)))
      return rc;
    rc = mp.hdim_is_batch ? permute_launch(h->d_a.ptr, h->d_a2.ptr, 1, 1, B, M, BL, K, h->stream)
                          : permute_launch(h->d_a.ptr, h->d_a2.ptr, 1, 0, 1, B, K, M, h->stream);
    if (rc)
      return rc;
    pa = (const uint8_t *)h->d_a2.ptr;
  }
  int gemm_rt = mp.right_transpose;  // [N, K] per batch is the layout the kernels read
  if (mp.right_transpose && mp.hdim_is_batch) {
    if ((rc = h->d_b2.reserve((size_t)b_num)) ||
        (rc = permute_launch(h->d_b.ptr, h->d_b2.ptr, 1, 1, B, K, BL, N, h->stream)))
      return rc;
    pb = (const uint8_t *)h->d_b2.ptr;
    gemm_rt = 0;  // the re-laid operand is [batch, batch_low, K, N]
  }
  const float *bias = p->n_inputs > 2 ? p->inputs[2] : nullptr;
  const float *multi = p->n_inputs > 3 ? p->inputs[3] : nullptr;
  if (bias && (rc = floats_to_i32_dev(bias, N, h->d_bias, h->stream)))
    return rc;
  const int64_t relu_limit = attr->relu_limit > 0.0 ? (int64_t)floor(attr->relu_limit) : -1;
  int32_t *acc = (int32_t *)h->d_acc.ptr;
  for (int64_t b = 0; b < FB; ++b) {
    rc = i8mm_launch(pa + b * M * K, a_unsigned, pb + b * K * N, b_unsigned, gemm_rt,
                     bias ? (const int32_t *)h->d_bias.ptr : nullptr, M, K, N, attr->input_zp, attr->right_zp,
                     attr->do_relu, relu_limit, nullptr, nullptr, acc + b * M * N, h->stream);
    if (rc)
      return rc;
  }
  if (mp.output_transpose) {
    if ((rc = h->d_acc2.reserve((size_t)o_num * 4)))
      return rc;
    rc = mp.hdim_is_batch ? permute_launch(acc, h->d_acc2.ptr, 4, 1, B, BL, M, N, h->stream)
                          : permute_launch(acc, h->d_acc2.ptr, 4, 0, B, BL, M, N, h->stream);
    if (rc)
      return rc;
    acc = (int32_t *)h->d_acc2.ptr;
  }
  const void *result = acc;
  if (attr->out_dtype != MI_DT_I32) {
    mi_requant_desc rq;
    fill_i8_rq(attr, &rq);
    int64_t outer = 1, channels = 1, inner = o_num;
    if (attr->chip == MI_CHIP_CV18XX) {
      if (FB > 1 && attr->n_multipliers == FB && attr->n_rshifts == FB) {  // MatMul.cpp:645-647: one pair per batch
        std::vector<int32_t> mb((size_t)FB), rb((size_t)FB);
        for (int64_t b = 0; b < FB; ++b) {
          mb[(size_t)b] = (int32_t)attr->multipliers[b];
          rb[(size_t)b] = (int32_t)attr->rshifts[b];
        }
        if ((rc = h->d_mult_b.reserve((size_t)FB * 4)) || (rc = h->d_rs_b.reserve((size_t)FB * 4)))
          return rc;
        MI_HIP(hipMemcpy(h->d_mult_b.ptr, mb.data(), (size_t)FB * 4, hipMemcpyHostToDevice));
        MI_HIP(hipMemcpy(h->d_rs_b.ptr, rb.data(), (size_t)FB * 4, hipMemcpyHostToDevice));
        rq.d_multiplier = (const int32_t *)h->d_mult_b.ptr;
        rq.d_shift = (const int32_t *)h->d_rs_b.ptr;
        channels = FB;
        inner = M * N;
      }
    } else if (attr->quant_mode == MI_RQ_MULTIPLIER_SHIFT && attr->fuse_rq) {
      MI_REQUIRE(multi, MI_BAD_ARGUMENT, "mi_i8mm_inference_nd: fuse_rq needs the multi operand");
      MI_REQUIRE(n_last > 0 && o_num % n_last == 0, MI_BAD_ARGUMENT, "mi_i8mm_inference_nd: bad output shape");
      if ((rc = floats_to_i32_dev(multi, n_last, h->d_multi, h->stream)))
        return rc;
      rq.d_multiplier = (const int32_t *)h->d_multi.ptr;
      outer = o_num / n_last;
      channels = n_last;
      inner = 1;
    }
    if ((rc = requant_launch(acc, h->d_out.ptr, outer, channels, inner, 0, &rq, h->stream)))
      return rc;
    result = h->d_out.ptr;
  }
  MI_HIP(hipMemcpyAsync(h->h_out.ptr, result, (size_t)o_num * osz, hipMemcpyDeviceToHost, h->stream));
  MI_HIP(hipStreamSynchronize(h->stream));
  bytes_to_floats(h->h_out.ptr, attr->out_dtype, o_num, p->outputs[0]);
  return MI_SUCCESS;
}

int mi_i8mm_inference_nd(const mi_i8mm_attr *attr, const mi_matmul_shapes *shapes, mi_infer_param *p) {
  MI_REQUIRE(attr && shapes && p, MI_BAD_ARGUMENT, "mi_i8mm_inference_nd: null argument");
  mi_matmul_param mp;
  int rc = mi_matmul_parse_param(shapes, attr->right_transpose, attr->chip, &mp);
  if (rc)
    return rc;
  const int64_t batch = mp.batch * mp.batch_low;
  int64_t a_num = 1, b_num = 1, o_num = 1;
  for (int i = 0; i < shapes->a_dims; ++i)
    a_num *= shapes->a_shape[i];
  for (int i = 0; i < shapes->b_dims; ++i)
    b_num *= shapes->b_shape[i];
  for (int i = 0; i < shapes->o_dims; ++i)
    o_num *= shapes->o_shape[i];
  MI_REQUIRE(a_num == batch * mp.M * mp.K && b_num == batch * mp.K * mp.N && o_num == batch * mp.M * mp.N,
             MI_UNSUPPORTED,
             "mi_i8mm_inference_nd: the operands do not hold exactly one matrix per batch (broadcast batches are not "
             "handled)");
  MI_REQUIRE(p->inputs && p->n_inputs >= 2 && p->inputs[0] && p->inputs[1] && p->outputs && p->n_outputs >= 1 &&
                 p->outputs[0],
             MI_BAD_ARGUMENT, "mi_i8mm_inference_nd: null input or output");
  if (mp.left_transpose || mp.output_transpose || mp.hdim_is_batch) {
    mi_i8mm_attr one = *attr;
    one.M = mp.M;
    one.K = mp.K;
    one.N = mp.N;
    if ((rc = check_i8_attr(&one, "mi_i8mm_inference_nd")))
      return rc;
    return i8mm_inference_relaid(attr, shapes, mp, p);
  }
  I8BatchHandle *bh = (I8BatchHandle *)p->handle;
  if (!bh) {
    bh = new I8BatchHandle;
    bh->per_batch.assign((size_t)batch, nullptr);
    p->handle = bh;
  }
  MI_REQUIRE(bh->magic == 0x18B18B18u && (int64_t)bh->per_batch.size() == batch, MI_BAD_ARGUMENT,
             "mi_i8mm_inference_nd: the handle belongs to another op or another batch size");
  const bool per_batch_q = attr->chip == MI_CHIP_CV18XX && batch > 1 && attr->n_multipliers == batch &&
                           attr->n_rshifts == batch;
  for (int64_t b = 0; b < batch; ++b) {
    mi_i8mm_attr one = *attr;
    one.M = mp.M;
    one.K = mp.K;
    one.N = mp.N;
    if (per_batch_q) {
      one.multipliers = attr->multipliers + b;
      one.n_multipliers = 1;
      one.rshifts = attr->rshifts + b;
      one.n_rshifts = 1;
    }
    const float *ins[5] = {p->inputs[0] + b * mp.M * mp.K, p->inputs[1] + b * mp.K * mp.N,
                           p->n_inputs > 2 ? p->inputs[2] : nullptr, p->n_inputs > 3 ? p->inputs[3] : nullptr, nullptr};
    float *outs[1] = {p->outputs[0] + b * mp.M * mp.N};
    mi_infer_param sub;
    sub.inputs = (float **)ins;
    sub.n_inputs = 5;
    sub.outputs = outs;
    sub.n_outputs = 1;
    sub.handle = bh->per_batch[(size_t)b];
    rc = mi_i8mm_inference(&one, &sub);
    bh->per_batch[(size_t)b] = sub.handle;
    if (rc)
      return rc;
  }
  return MI_SUCCESS;
}

// ---------------------------------------------------------------------------------------------
// operator level: tpu.RequantIntAxis / tpu.RequantInt
// ---------------------------------------------------------------------------------------------
static int run_requant_host(const float *in, float *out, int64_t outer, int64_t channels, int64_t inner,
                            int64_t input_zp, mi_requant_desc rq, const std::vector<int32_t> *mult,
                            const std::vector<int32_t> *shift, const std::vector<int32_t> *zp) {
  MI_REQUIRE(mi_device_count() > 0, MI_HIP_ERROR, "requant: no GPU visible");
  const int64_t total = outer * channels * inner;
  const int osz = out_elem_size(rq.out_dtype);
  std::vector<int32_t> hin((size_t)total);
  for (int64_t i = 0; i < total; ++i)
    hin[(size_t)i] = (int32_t)(int64_t)in[i];
  DevBuf d_in, d_out, d_m, d_s, d_z;
  int rc;
  if ((rc = d_in.reserve((size_t)total * 4)) || (rc = d_out.reserve((size_t)total * osz)))
    return rc;
  MI_HIP(hipMemcpy(d_in.ptr, hin.data(), (size_t)total * 4, hipMemcpyHostToDevice));
  if (mult) {
    if ((rc = d_m.reserve(mult->size() * 4)) || (rc = d_s.reserve(shift->size() * 4)) ||
        (rc = d_z.reserve(zp->size() * 4)))
      return rc;
    MI_HIP(hipMemcpy(d_m.ptr, mult->data(), mult->size() * 4, hipMemcpyHostToDevice));
    MI_HIP(hipMemcpy(d_s.ptr, shift->data(), shift->size() * 4, hipMemcpyHostToDevice));
    MI_HIP(hipMemcpy(d_z.ptr, zp->data(), zp->size() * 4, hipMemcpyHostToDevice));
    rq.d_multiplier = (const int32_t *)d_m.ptr;
    rq.d_shift = (const int32_t *)d_s.ptr;
    rq.d_zp = (const int32_t *)d_z.ptr;
  }
  if ((rc = requant_launch((const int32_t *)d_in.ptr, d_out.ptr, outer, channels, inner, input_zp, &rq, nullptr)))
    return rc;
  std::vector<uint8_t> hout((size_t)total * osz);
  MI_HIP(hipMemcpy(hout.data(), d_out.ptr, hout.size(), hipMemcpyDeviceToHost));
  for (int64_t i = 0; i < total; ++i) {
    switch (rq.out_dtype) {
    case MI_DT_I8: out[i] = (float)((const int8_t *)hout.data())[i]; break;
    case MI_DT_U8: out[i] = (float)((const uint8_t *)hout.data())[i]; break;
    case MI_DT_I16: out[i] = (float)((const int16_t *)hout.data())[i]; break;
    case MI_DT_U16: out[i] = (float)((const uint16_t *)hout.data())[i]; break;
    default: out[i] = (float)((const int32_t *)hout.data())[i]; break;
    }
  }
  return MI_SUCCESS;
}

int mi_requant_int_axis_inference(const mi_rq_axis_attr *a, mi_infer_param *p) {
  MI_REQUIRE(a && p && p->inputs && p->n_inputs >= 2 && p->inputs[0] && p->inputs[1] && p->outputs &&
                 p->n_outputs >= 1 && p->outputs[0],
             MI_BAD_ARGUMENT, "mi_requant_int_axis_inference: null argument");
  MI_REQUIRE(a->rank >= 2 && a->rank <= 8, MI_BAD_ARGUMENT, "mi_requant_int_axis_inference: bad rank");
  const int q = a->quant_mode;
  MI_REQUIRE(q == MI_RQ_TFLITE || q == MI_RQ_TFLITE_LSHIFT || q == MI_RQ_MULTIPLIER_SHIFT, MI_UNSUPPORTED,
             "mi_requant_int_axis_inference: requant mode not handled");
  const bool tflite = q != MI_RQ_MULTIPLIER_SHIFT;
  const bool last_axis = !tflite && a->fuse_rq_axis;
  int64_t outer, channels, inner;
  if (last_axis) {  // RequantIntAxis.cpp:68-91
    channels = a->shape[a->rank - 1];
    inner = 1;
    outer = 1;
    for (int i = 0; i < a->rank - 1; ++i)
      outer *= a->shape[i];
  } else {  // :41-66, :93-118: channel = dim 1
    outer = a->shape[0];
    channels = a->shape[1];
    inner = 1;
    for (int i = 2; i < a->rank; ++i)
      inner *= a->shape[i];
  }
  const float *quant = p->inputs[1];
  std::vector<int32_t> mult((size_t)channels), shift((size_t)channels), zp((size_t)channels);
  for (int64_t c = 0; c < channels; ++c) {
    int64_t m, s, z;
    if (a->quant_triples) {
      m = (int64_t)quant[c * 3];
      s = (int64_t)quant[c * 3 + 1];
      z = (int64_t)quant[c * 3 + 2];
    } else {  // :50-55: shift in the low byte, zero point in the high half-word
      m = (int64_t)quant[c * 2];
      uint32_t tmp = (uint32_t)quant[c * 2 + 1];
      s = (int64_t)((signed char)(tmp & 0xff));
      z = (int64_t)(short)((tmp & 0xffff0000u) >> 16);
    }
    // device convention: positive = right shift.  The TFLite branch hands the stored shift to
    // MultiplyByQuantizedMultiplier (negative = right); the axis-1 MultiplierShift branch negates the stored
    // value into a right shift; the fused-axis branch uses it as a right shift directly.
    int64_t rs = (tflite || !last_axis) ? -s : s;
    mult[(size_t)c] = (int32_t)m;
    shift[(size_t)c] = (int32_t)rs;
    zp[(size_t)c] = (int32_t)z;
  }
  mi_requant_desc rq;
  memset(&rq, 0, sizeof(rq));
  rq.quant_mode = q;
  rq.round_mode = a->round_mode;
  rq.chip = a->chip;
  rq.out_dtype = a->out_dtype;
  return run_requant_host(p->inputs[0], p->outputs[0], outer, channels, inner, tflite ? 0 : a->input_zp, rq, &mult,
                          &shift, &zp);
}

int mi_requant_int_inference(const mi_rq_attr *a, mi_infer_param *p) {
  MI_REQUIRE(a && p && p->inputs && p->n_inputs >= 1 && p->inputs[0] && p->outputs && p->n_outputs >= 1 &&
                 p->outputs[0],
             MI_BAD_ARGUMENT, "mi_requant_int_inference: null argument");
  MI_REQUIRE(a->rank >= 1 && a->rank <= 8, MI_BAD_ARGUMENT, "mi_requant_int_inference: bad rank");
  if (a->rank == 1)
    return MI_SUCCESS;  // RequantInt.cpp:36-38
  const int q = a->quant_mode;
  MI_REQUIRE(q == MI_RQ_TFLITE || q == MI_RQ_TFLITE_LSHIFT || q == MI_RQ_MULTIPLIER_SHIFT, MI_UNSUPPORTED,
             "mi_requant_int_inference: requant mode not handled");
  int64_t total = 1;
  for (int i = 0; i < a->rank; ++i)
    total *= a->shape[i];
  mi_requant_desc rq;
  memset(&rq, 0, sizeof(rq));
  rq.quant_mode = q;
  rq.round_mode = a->round_mode;
  rq.chip = a->chip;
  rq.out_dtype = a->out_dtype;
  rq.multiplier = (int32_t)a->multiplier;
  rq.shift = (int32_t)a->rshift;  // both branches shift right by getRshift() (RequantInt.cpp:31,47,62)
  rq.zp = (int32_t)a->out_zp;
  return run_requant_host(p->inputs[0], p->outputs[0], 1, 1, total, q == MI_RQ_MULTIPLIER_SHIFT ? a->input_zp : 0, rq,
                          nullptr, nullptr, nullptr);
}

// ---------------------------------------------------------------------------------------------
// tpu.Cast
// ---------------------------------------------------------------------------------------------
static bool st_float(int t) { return t == MI_ST_F32 || t == MI_ST_BF16 || t == MI_ST_F16; }

// the scalars the reference forms once per call: (float)(1.0 / scale) narrowed to the expressed type
// (CastUtils.cpp:18-27) and the scale narrowed to the output type of a dequantizing cast (Cast.cpp:107-117)
}  // extern "C"
namespace mi {
int cast_scalars(const mi_cast_attr *a, float *inv_scale, float *scale) {
  MI_REQUIRE(a, MI_BAD_ARGUMENT, "mi_cast: null attribute");
  MI_REQUIRE(a->in_type >= MI_ST_F32 && a->in_type <= MI_ST_F8E5M2 && a->out_type >= MI_ST_F32 &&
                 a->out_type <= MI_ST_F8E5M2,
             MI_UNSUPPORTED, "mi_cast: storage type not handled");
  {  // 8-bit floats: from and to F32 / F16 only, never quantized (Cast.cpp:59-73)
    const bool f8_in = a->in_type >= MI_ST_F8E4M3, f8_out = a->out_type >= MI_ST_F8E4M3;
    const bool wide_in = a->in_type == MI_ST_F32 || a->in_type == MI_ST_F16;
    const bool wide_out = a->out_type == MI_ST_F32 || a->out_type == MI_ST_F16;
    MI_REQUIRE((!f8_in && !f8_out) || (f8_out && wide_in && !a->in_quant && !a->out_quant) ||
                   (f8_in && wide_out && !a->in_quant && !a->out_quant),
               MI_UNSUPPORTED, "mi_cast: an 8-bit float casts from and to F32 / F16 only");
  }
  MI_REQUIRE(a->chip == MI_CHIP_BM168X || a->chip == MI_CHIP_CV18XX || a->chip == MI_CHIP_BM1684, MI_BAD_ARGUMENT,
             "mi_cast: unknown chip");
  MI_REQUIRE(a->num_elem >= 0, MI_BAD_ARGUMENT, "mi_cast: negative element count");
  *inv_scale = 1.0f;
  *scale = (float)a->scale;
  if (a->chip == MI_CHIP_CV18XX) {
    // Cast.cpp:82-84, :18-26: BF16(1. / scale) and BF16(scale) with the chip's rounding (add 0x7fff + lsb, truncate,
    // an all-ones exponent becomes 0x7f7f: Float16.cpp:725-761)
    MI_REQUIRE(a->in_type < MI_ST_F8E4M3 && a->out_type < MI_ST_F8E4M3, MI_UNSUPPORTED,
               "mi_cast: 8-bit floats are not handled for CV18xx");
    auto cvi = [](float f) {
      uint32_t u = fbits(f);
      u += 0x7fffu + ((u >> 16) & 1u);
      uint32_t h = u >> 16;
      if ((h & 0x7f80u) == 0x7f80u)
        h = 0x7f7fu;
      return bits_f(h << 16);
    };
    if (a->out_quant && st_float(a->in_type)) {
      MI_REQUIRE(a->scale != 0.0 && a->scale == a->scale, MI_BAD_ARGUMENT, "mi_cast: scale must be a nonzero number");
      *inv_scale = cvi((float)(1. / a->scale));
    } else if (a->in_quant && st_float(a->out_type)) {
      *scale = cvi((float)a->scale);
    }
    return MI_SUCCESS;
  }
  const bool quantizing = a->out_quant && st_float(a->in_type);
  const bool dequantizing = !quantizing && a->in_quant && st_float(a->out_type);
  if (quantizing || dequantizing)
    MI_REQUIRE(a->scale != 0.0 && a->scale == a->scale, MI_BAD_ARGUMENT, "mi_cast: scale must be a nonzero number");
  if (quantizing) {
    MI_REQUIRE(a->expressed == MI_ST_F32 || a->expressed == MI_ST_BF16 || a->expressed == MI_ST_F16,
               MI_UNSUPPORTED, "mi_cast: expressed type not handled");
    float inv = (float)(1.0 / a->scale);
    if (a->expressed == MI_ST_F16)
      inv = h_f16_to_f32(h_f32_to_f16(inv));
    else if (a->expressed == MI_ST_BF16)
      inv = h_bf16_to_f32(h_f32_to_bf16(inv));
    *inv_scale = inv;
  }
  if (dequantizing) {
    if (a->out_type == MI_ST_F16)
      *scale = h_f16_to_f32(h_f32_to_f16((float)a->scale));
    else if (a->out_type == MI_ST_BF16)
      *scale = h_bf16_to_f32(h_f32_to_bf16((float)a->scale));
  }
  return MI_SUCCESS;
}
}  // namespace mi
extern "C" {

int mi_cast_launch(const mi_cast_attr *a, const void *d_in, void *d_out, void *stream) {
  float inv, sc;
  int rc = cast_scalars(a, &inv, &sc);
  if (rc)
    return rc;
  MI_REQUIRE(a->num_elem == 0 || (d_in && d_out), MI_BAD_ARGUMENT, "mi_cast_launch: null operand");
  return cast_launch(a, d_in, d_out, a->num_elem, inv, sc, false, (hipStream_t)stream);
}

int mi_cast_inference(const mi_cast_attr *a, mi_infer_param *p) {
  MI_REQUIRE(a && p && p->inputs && p->n_inputs >= 1 && p->inputs[0] && p->outputs && p->n_outputs >= 1 &&
                 p->outputs[0],
             MI_BAD_ARGUMENT, "mi_cast_inference: null argument");
  float inv, sc;
  int rc = cast_scalars(a, &inv, &sc);
  if (rc)
    return rc;
  MI_REQUIRE(mi_device_count() > 0, MI_HIP_ERROR, "mi_cast_inference: no GPU visible");
  const int64_t n = a->num_elem;
  // the interpreter's tensors are float arrays whatever the storage type: both sides travel as f32 here and the
  // kernel applies the op's arithmetic between them
  DevBuf d_in, d_out;
  if ((rc = d_in.reserve((size_t)n * 4 + 4)) || (rc = d_out.reserve((size_t)n * 4 + 4)))
    return rc;
  MI_HIP(hipMemcpy(d_in.ptr, p->inputs[0], (size_t)n * 4, hipMemcpyHostToDevice));
  rc = cast_launch(a, d_in.ptr, d_out.ptr, n, inv, sc, true, nullptr);
  if (rc)
    return rc;
  MI_HIP(hipMemcpy(p->outputs[0], d_out.ptr, (size_t)n * 4, hipMemcpyDeviceToHost));
  return MI_SUCCESS;
}

// ---- tpu.MatMul on F8E4M3 operands with F8 output requantization (MatMul.cpp:598-629) --------------------------
int mi_f8mm_launch(const uint8_t *d_a, const uint8_t *d_b, int right_transpose, const float *d_bias, int64_t M,
                   int64_t K, int64_t N, int do_relu, double relu_limit, double out_scale, const double *d_out_scales,
                   int out_kind, void *d_out, float *d_acc_f32, void *stream) {
  return f8mm_launch(d_a, d_b, right_transpose, d_bias, M, K, N, do_relu, relu_limit, out_scale, d_out_scales, out_kind,
                     d_out, d_acc_f32, (hipStream_t)stream);
}

int mi_f8mm_e5m2_launch(const uint8_t *d_a, const uint8_t *d_b, int right_transpose, const float *d_bias, int64_t M,
                        int64_t K, int64_t N, int do_relu, double relu_limit, int out_kind, void *d_out,
                        float *d_acc_f32, void *stream) {
  return f8mm_launch(d_a, d_b, right_transpose, d_bias, M, K, N, do_relu, relu_limit, 1.0, nullptr, out_kind, d_out,
                     d_acc_f32, (hipStream_t)stream, MI_F8_E5M2);
}

// f32 -> the E5M2 code of exactly that value (finite values only), or -1: an E5M2 value is a half whose low byte is 0
static int f8e5m2_code_of(float v) {
  uint32_t b;
  memcpy(&b, &v, 4);
  const uint32_t sign = (b >> 24) & 0x80u, a = b & 0x7fffffffu;
  if (a == 0)
    return (int)sign;
  const int e = (int)(a >> 23) - 127;
  const uint32_t frac = a & 0x7fffffu;
  if (e >= -14 && e <= 15) {           // normals: 2 fraction bits
    if (frac & 0x1fffffu)
      return -1;
    return (int)((((uint32_t)(e + 15) << 2) | (frac >> 21)) | sign);
  }
  if (e >= -16 && e < -14) {           // subnormals: multiples of 2^-16 below 2^-14
    const uint32_t mant = frac | 0x800000u;
    const int shift = 23 - (e + 16);
    if (mant & ((1u << shift) - 1))
      return -1;
    return (int)((mant >> shift) | sign);
  }
  return -1;
}

// f32 -> the E4M3 code of exactly that value, or -1 (host side of the operator entry: the interpreter hands over
// f32 arrays that hold E4M3 values)
static int f8_code_of(float v) {
  uint32_t b;
  memcpy(&b, &v, 4);
  const uint32_t sign = (b >> 24) & 0x80u, a = b & 0x7fffffffu;
  if (a == 0)
    return (int)sign;
  const int e = (int)(a >> 23) - 127;  // unbiased
  const uint32_t frac = a & 0x7fffffu;
  if (e >= -6 && e <= 8) {             // E4M3 normals: 3 fraction bits
    if (frac & 0xfffffu)
      return -1;
    const uint32_t code = ((uint32_t)(e + 7) << 3) | (frac >> 20);
    return code >= 0x7f ? -1 : (int)(code | sign);
  }
  if (e >= -9 && e < -6) {             // subnormals: multiples of 2^-9 below 2^-6
    const uint32_t mant = (frac | 0x800000u);  // 1.f at bit 23, value = mant * 2^(e - 23)
    const int shift = 23 - (e + 9);            // units of 2^-9
    if (mant & ((1u << shift) - 1))
      return -1;
    return (int)((mant >> shift) | sign);
  }
  return -1;
}

int mi_f8mm_inference(const mi_f8mm_attr *a, mi_infer_param *p) {
  MI_REQUIRE(a && p && p->inputs && p->n_inputs >= 2 && p->inputs[0] && p->inputs[1] && p->outputs &&
                 p->n_outputs >= 1 && p->outputs[0],
             MI_BAD_ARGUMENT, "mi_f8mm_inference: null argument");
  MI_REQUIRE(a->M >= 0 && a->K > 0 && a->N > 0, MI_BAD_ARGUMENT, "mi_f8mm_inference: bad shape");
  MI_REQUIRE(a->f8_type == MI_F8_E4M3 || a->f8_type == MI_F8_E5M2, MI_BAD_ARGUMENT, "mi_f8mm_inference: f8_type");
  const bool e5m2 = a->f8_type == MI_F8_E5M2;
  MI_REQUIRE(e5m2 || (a->out_scales && (a->n_out_scales == 1 || a->n_out_scales == a->N)), MI_BAD_ARGUMENT,
             "mi_f8mm_inference: out_scales must hold one scale or one per output channel");
  for (int i = 0; !e5m2 && i < a->n_out_scales; ++i)
    MI_REQUIRE(a->out_scales[i] == a->out_scales[i] && a->out_scales[i] != 0.0, MI_BAD_ARGUMENT,
               "mi_f8mm_inference: output scales must be nonzero numbers");
  if (a->M == 0)
    return MI_SUCCESS;
  MI_REQUIRE(mi_device_count() > 0, MI_HIP_ERROR, "mi_f8mm_inference: no GPU visible");
  const size_t nl = (size_t)a->M * a->K, nr = (size_t)a->K * a->N, no = (size_t)a->M * a->N;
  std::vector<uint8_t> hl(nl), hr(nr);
  for (size_t i = 0; i < nl; ++i) {
    const int c = e5m2 ? f8e5m2_code_of(p->inputs[0][i]) : f8_code_of(p->inputs[0][i]);
    MI_REQUIRE(c >= 0, MI_UNSUPPORTED, "mi_f8mm_inference: left operand holds a value that is not a finite number of its 8-bit type");
    hl[i] = (uint8_t)c;
  }
  for (size_t i = 0; i < nr; ++i) {
    const int c = e5m2 ? f8e5m2_code_of(p->inputs[1][i]) : f8_code_of(p->inputs[1][i]);
    MI_REQUIRE(c >= 0, MI_UNSUPPORTED, "mi_f8mm_inference: right operand holds a value that is not a finite number of its 8-bit type");
    hr[i] = (uint8_t)c;
  }
  const float *bias = p->n_inputs > 2 ? p->inputs[2] : nullptr;
  DevBuf dl, dr, db, ds, dy;
  int rc;
  if ((rc = dl.reserve(nl)) || (rc = dr.reserve(nr)) || (rc = dy.reserve(no * 4)))
    return rc;
  MI_HIP(hipMemcpy(dl.ptr, hl.data(), nl, hipMemcpyHostToDevice));
  MI_HIP(hipMemcpy(dr.ptr, hr.data(), nr, hipMemcpyHostToDevice));
  if (bias) {
    if ((rc = db.reserve((size_t)a->N * 4)))
      return rc;
    MI_HIP(hipMemcpy(db.ptr, bias, (size_t)a->N * 4, hipMemcpyHostToDevice));
  }
  if (!e5m2 && a->n_out_scales != 1) {
    if ((rc = ds.reserve((size_t)a->N * 8)))
      return rc;
    MI_HIP(hipMemcpy(ds.ptr, a->out_scales, (size_t)a->N * 8, hipMemcpyHostToDevice));
  }
  rc = f8mm_launch((const uint8_t *)dl.ptr, (const uint8_t *)dr.ptr, a->right_transpose, bias ? (const float *)db.ptr : nullptr,
                   a->M, a->K, a->N, a->do_relu, a->relu_limit, e5m2 ? 1.0 : a->out_scales[0],
                   !e5m2 && a->n_out_scales != 1 ? (const double *)ds.ptr : nullptr, MI_F8_OUT_F32, dy.ptr, nullptr,
                   nullptr, a->f8_type);
  if (rc)
    return rc;
  MI_HIP(hipDeviceSynchronize());
  MI_HIP(hipMemcpy(p->outputs[0], dy.ptr, no * 4, hipMemcpyDeviceToHost));
  return MI_SUCCESS;
}

// ---- tpu.MatMul, both operands quantized dynamically (MatMul.cpp:447-597) -------------------------------------
int mi_matmul_dq_launch(const uint16_t *d_left, const uint16_t *d_right, int right_transpose, int64_t M, int64_t K,
                        int64_t N, int q_group_size, int dq_type, int dtype, uint16_t *d_y, float *d_y_f32,
                        void *stream) {
  return matmul_dq_launch(d_left, d_right, right_transpose, M, K, N, q_group_size, dq_type, dtype, d_y, d_y_f32,
                          (hipStream_t)stream);
}

int mi_matmul_dq_inference(const mi_matmul_dq_attr *a, mi_infer_param *p) {
  MI_REQUIRE(a && p && p->inputs && p->n_inputs >= 2 && p->inputs[0] && p->inputs[1] && p->outputs &&
                 p->n_outputs >= 1 && p->outputs[0],
             MI_BAD_ARGUMENT, "mi_matmul_dq_inference: null argument");
  MI_REQUIRE(a->M >= 0 && a->K > 0 && a->N > 0, MI_BAD_ARGUMENT, "mi_matmul_dq_inference: bad shape");
  MI_REQUIRE(a->dq_type == MI_DQ_INT8 || a->dq_type == MI_DQ_INT4 || a->dq_type == MI_DQ_F8E4M3 || a->dq_type == MI_DQ_F4,
             MI_UNSUPPORTED, "mi_matmul_dq_inference: dq_type must be MI_DQ_INT8, MI_DQ_INT4, MI_DQ_F8E4M3 or MI_DQ_F4");
  MI_REQUIRE(a->out_dtype == MI_DT_BF16 || a->out_dtype == MI_DT_F16, MI_UNSUPPORTED, "mi_matmul_dq_inference: out_dtype");
  const int64_t g = a->q_group_size == -1 ? a->K : a->q_group_size;
  MI_REQUIRE(g > 0, MI_BAD_ARGUMENT, "mi_matmul_dq_inference: dynamic quantization needs a group size");
  if (a->M == 0)
    return MI_SUCCESS;
  MI_REQUIRE(mi_device_count() > 0, MI_HIP_ERROR, "mi_matmul_dq_inference: no GPU visible");
  const bool f16 = a->out_dtype == MI_DT_F16;
  const size_t nl = (size_t)a->M * a->K, nr = (size_t)a->K * a->N, no = (size_t)a->M * a->N;
  // the operands are activations in the 16-bit type (f32-valued on the host side)
  std::vector<uint16_t> hl(nl), hr(nr), ho(no);
  for (size_t i = 0; i < nl; ++i)
    hl[i] = f16 ? h_f32_to_f16(p->inputs[0][i]) : h_f32_to_bf16(p->inputs[0][i]);
  for (size_t i = 0; i < nr; ++i)
    hr[i] = f16 ? h_f32_to_f16(p->inputs[1][i]) : h_f32_to_bf16(p->inputs[1][i]);
  DevBuf dl, dr, dy;
  int rc;
  if ((rc = dl.reserve(nl * 2)) || (rc = dr.reserve(nr * 2)) || (rc = dy.reserve(no * 2)))
    return rc;
  MI_HIP(hipMemcpy(dl.ptr, hl.data(), nl * 2, hipMemcpyHostToDevice));
  MI_HIP(hipMemcpy(dr.ptr, hr.data(), nr * 2, hipMemcpyHostToDevice));
  rc = matmul_dq_launch((const uint16_t *)dl.ptr, (const uint16_t *)dr.ptr, a->right_transpose, a->M, a->K, a->N,
                        a->q_group_size, a->dq_type, a->out_dtype, (uint16_t *)dy.ptr, nullptr, nullptr);
  if (rc)
    return rc;
  MI_HIP(hipDeviceSynchronize());
  MI_HIP(hipMemcpy(ho.data(), dy.ptr, no * 2, hipMemcpyDeviceToHost));
  for (size_t i = 0; i < no; ++i)
    p->outputs[0][i] = f16 ? h_f16_to_f32(ho[i]) : h_bf16_to_f32(ho[i]);
  return MI_SUCCESS;
}

}  // extern "C"
