// extern "C" surface of libcpnsort.so (declared in include/cpn_sort.h): argument checks,
// dtype dispatch and the status read-back.  Plays the role of local_sort<CODE>
// (src/cupynumeric/sort/sort.cu:63-96) plus the type dispatch of sort_template
// (src/cupynumeric/sort/sort_template.inl:92-120).
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <atomic>
#include <mutex>

#include "sort_driver.h"

// Device memory for cpn_local_sort_static: the workspace of a sort that may not allocate.  One
// copy of the array exists on every GPU that loads this library, for the life of the process.
// In host code the name below is only a handle for hipGetSymbolAddress; kernels and HIP calls
// receive the per-device address kept in g_static_scratch.
static __device__ __align__(256) unsigned char scratch[CPN_STATIC_SCRATCH_BYTES];

namespace cpn {

thread_local int g_last_hip_error = 0;

int swapaxes_copy(int elem_bytes, const void* in, void* out, const int64_t* shape, int ndim, int axis_a, int axis_b,
                  hipStream_t stream);

// -1 = not overridden.  Initialised from CPN_SORT_LDS_ROW_LIMIT, changed by cpn_set_lds_row_limit.
static std::atomic<long long> g_lds_row_limit{[] {
  const char* e = getenv("CPN_SORT_LDS_ROW_LIMIT");
  return (e != nullptr && *e != 0) ? atoll(e) : -1ll;
}()};

// Longest row given to the one-wavefront-per-row kernel (0 = never).
static std::atomic<long long> g_wave_row_limit{[] {
  const char* e = getenv("CPN_SORT_WAVE_ROW_LIMIT");
  return (e != nullptr && *e != 0) ? atoll(e) : 1024ll;
}()};

// Rows from this length on take the 64-bit variant of the global kernels (never above 2^30).
static std::atomic<long long> g_wide_row_threshold{[] {
  const char* e = getenv("CPN_SORT_WIDE_ROW_THRESHOLD");
  return (e != nullptr && *e != 0) ? atoll(e) : -1ll;
}()};

uint64_t wide_row_threshold()
{
  const long long t = g_wide_row_threshold.load(std::memory_order_relaxed);
  return (t < 0 || static_cast<uint64_t>(t) > BIG_ROW_ELEMENTS) ? BIG_ROW_ELEMENTS : static_cast<uint64_t>(t);
}

// 0: tiles dealt per XCD, 1: one ticket counter for the launch
static std::atomic<int> g_tile_order{[] {
  const char* e = getenv("CPN_SORT_TILE_ORDER");
  return (e != nullptr && (e[0] == 's' || e[0] == '1')) ? 1 : 0;
}()};

bool tile_order_single() { return g_tile_order.load(std::memory_order_relaxed) != 0; }

// Rows longer than the LDS capacity, sorted in pieces and merged: 0 = never (global path), 1 = up to the
// built-in number of levels of merging per key width, N >= 2 = up to N - 1 levels whatever the key (A/B runs)
static std::atomic<int> g_merge_rows{[] {
  const char* e = getenv("CPN_SORT_MERGE_ROWS");
  const int v   = (e != nullptr && *e != 0) ? atoi(e) : 1;
  return v < 0 ? 1 : v;
}()};

bool merge_rows_enabled() { return g_merge_rows.load(std::memory_order_relaxed) != 0; }

// Measured on 2^26 keys: a level of merging costs 0.17 ms for 4-byte keys (0.27 with positions) and
// 0.25 ms for 8-byte keys (0.41 with positions) on top of 0.46 (0.67) and 0.72 (0.70) ms for the
// pieces; the global path 0.92 (1.26) ms with its 4 passes and 2.7 (3.3) ms with its 8.
int merge_levels_limit(int key_bytes, bool want_indices)
{
  const int v = g_merge_rows.load(std::memory_order_relaxed);
  if (v >= 2) {
    return v - 1;
  }
  return key_bytes == 8 ? (want_indices ? 5 : 6) : 2;
}

// 1: short rows of real keys (2 ... bitonic_row_limit keys) go through the sorting network; 0: through the ranking kernels
static std::atomic<int> g_bitonic_rows{[] {
  const char* e = getenv("CPN_SORT_BITONIC_ROWS");
  return (e != nullptr && e[0] == '0') ? 0 : 1;
}()};

bool bitonic_rows_enabled() { return g_bitonic_rows.load(std::memory_order_relaxed) != 0; }
uint64_t bitonic_row_limit(int key_bytes, bool with_positions, bool float_keys)
{
  static const uint64_t cap = [] {
    const char* e = getenv("CPN_SORT_BITONIC_ROW_LIMIT");
    return e != nullptr && *e != '\0' ? strtoull(e, nullptr, 10) : ~0ull;
  }();
  // Measured on 2^26 keys against the kernels that take over (network / other, ms).  Values only: float16 rows of
  // 257 0.23 / 0.30, of 512 0.16 / 0.19; int16 rows of 257 0.22 / 0.27; float32 rows of 257 0.26 / 0.35, of 512
  // 0.18 / 0.23; float64 rows of 129 0.29 / 0.51, of 256 0.26 / 0.33, of 257 0.36 / 0.40, of 512 0.30 / 0.28; int64
  // rows of 256 0.31 / 0.33, of 257 0.45 / 0.40; int8 rows of 129 0.29 / 0.18, of 256 0.11 / 0.11.  With
  // positions: float16 rows of 257 0.29 / 0.43, of 512 0.19 / 0.27; float32 rows of 257 0.33 / 0.41, of 512 0.27 /
  // 0.30; float64 rows of 129 0.50 / 0.49, of 256 0.42 / 0.36.  A row per wavefront with up to 16 elements per
  // lane, 513 ... 1024 keys: float32 rows of 513 0.26 / 0.25, of 640 0.22 / 0.25, of 896 0.24 / 0.27, of 1024
  // 0.23 / 0.25 (int32 0.26 / 0.23, 0.22 / 0.22, 0.23 / 0.25, 0.21 / 0.23), with positions 0.34 / 0.35, 0.30 /
  // 0.33, 0.30 / 0.32, 0.29 / 0.32; float16 rows of 513 0.24 / 0.28, of 768 0.20 / 0.21, of 896 0.22 / 0.19, of
  // 1024 0.18 / 0.18, with positions 0.28 / 0.42, 0.25 / 0.32, 0.27 / 0.29, 0.23 / 0.27.  float64, values only, 32
  // lanes of 10 ... 16: rows of 257 0.36 / 0.42, of 384 0.30 / 0.35, of 448 0.32 / 0.31, of 500 0.34 / 0.31.
  uint64_t limit = 128;
  if (key_bytes == 2 || key_bytes == 4) {
    limit = (key_bytes == 2 && !with_positions) ? 768 : 1024;
  } else if (key_bytes == 1) {
    limit = with_positions ? 256 : 128;
  } else if (!with_positions) {
    limit = float_keys ? 384 : 256;  // (8-byte keys; float64 keys are compared as numbers)
  }
  return limit < cap ? limit : cap;
}

static std::atomic<long long> g_spin_limit{static_cast<long long>(LOOKBACK_SPIN_LIMIT)};

uint32_t lookback_spin_limit() { return static_cast<uint32_t>(g_spin_limit.load(std::memory_order_relaxed)); }

static std::atomic<long long> g_virt_threshold{[] {
  const char* e = getenv("CPN_SORT_VIRTUAL_DIGIT_THRESHOLD");
  return (e != nullptr && *e != 0) ? atoll(e) : static_cast<long long>(VIRT_MIN_ROW_ELEMENTS);
}()};

uint64_t virtual_digit_threshold() { return static_cast<uint64_t>(g_virt_threshold.load(std::memory_order_relaxed)); }

static const long long g_count16_min_row = [] {
  const char* e = getenv("CPN_SORT_COUNT16_MIN_ROW");
  return (e != nullptr && *e != 0) ? atoll(e) : static_cast<long long>(COUNT16_MIN_ROW);
}();

uint64_t count16_min_row() { return g_count16_min_row < 0 ? 0 : static_cast<uint64_t>(g_count16_min_row); }


uint64_t wave_row_limit()
{
  const long long limit = g_wave_row_limit.load(std::memory_order_relaxed);
  return limit < 0 ? 0 : (limit > 1024 ? 1024 : static_cast<uint64_t>(limit));
}

uint64_t lds_row_limit(int key_bytes, bool with_positions)
{
  const long long limit = g_lds_row_limit.load(std::memory_order_relaxed);
  uint64_t cap          = lds_row_capacity(key_bytes, with_positions);
  if (key_bytes == 2 && !with_positions && count16_min_row() <= cap + 1) {
    cap = COUNT16_ROW_CAPACITY;  // the counting kernel takes over where the radix shapes end
  }
  if (limit >= 0 && static_cast<uint64_t>(limit) < cap) {
    return static_cast<uint64_t>(limit);
  }
  return cap;
}

// Address of `scratch` on every device seen so far (looked up once per device, with that device
// current).
constexpr int MAX_DEVICES = 64;
static void* g_static_scratch[MAX_DEVICES];
static std::mutex g_static_scratch_mutex;

static int static_scratch_of_current_device(void** out)
{
  int dev = -1;
  CPN_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= MAX_DEVICES) {
    return CPN_ERR_UNSUPPORTED;
  }
  std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
  if (g_static_scratch[dev] == nullptr) {
    void* ptr = nullptr;
    CPN_HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (ptr == nullptr || (reinterpret_cast<uintptr_t>(ptr) % WORKSPACE_ALIGN) != 0) {
      return CPN_ERR_TEMP;
    }
    g_static_scratch[dev] = ptr;
  }
  *out = g_static_scratch[dev];
  return CPN_OK;
}

// one thread: hands the status word of a finished sort to the caller's device memory
static __global__ void copy_status_kernel(const uint32_t* __restrict__ status, uint32_t* __restrict__ out)
{
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    *out = *status;
  }
}

}  // namespace cpn

extern "C" {

int cpn_sort_version(void) { return (0 << 16) | 1; }

const char* cpn_status_string(int status)
{
  switch (status) {
    case CPN_OK: return "ok";
    case CPN_ERR_DTYPE: return "unknown element type code";
    case CPN_ERR_NULL: return "required pointer is NULL";
    case CPN_ERR_SHAPE: return "sort_dim_size is zero or does not divide volume, or bad axes";
    case CPN_ERR_TEMP: return "workspace missing, too small or not 256-byte aligned";
    case CPN_ERR_ALIGN: return "data pointer is not aligned to its element size";
    case CPN_ERR_HIP: return "HIP runtime call failed";
    case CPN_ERR_DEVICE: return "kernel reported an internal failure";
    case CPN_ERR_UNSUPPORTED: return "request not implemented by this build";
    case CPN_ERR_SCRATCH: return "request needs more workspace than the static scratch holds";
    default: return "unknown status";
  }
}

int cpn_last_hip_error(void) { return cpn::g_last_hip_error; }

int64_t cpn_set_lds_row_limit(int64_t limit)
{
  return static_cast<int64_t>(cpn::g_lds_row_limit.exchange(limit < 0 ? -1ll : static_cast<long long>(limit)));
}

int64_t cpn_set_wide_row_threshold(int64_t elements)
{
  return static_cast<int64_t>(cpn::g_wide_row_threshold.exchange(elements < 0 ? -1ll : static_cast<long long>(elements)));
}

int64_t cpn_set_virtual_digit_threshold(int64_t elements)
{
  const long long v = elements < 0 ? static_cast<long long>(cpn::VIRT_MIN_ROW_ELEMENTS) : static_cast<long long>(elements);
  return static_cast<int64_t>(cpn::g_virt_threshold.exchange(v));
}

int64_t cpn_set_lookback_spin_limit(int64_t polls)
{
  const long long v = (polls < 1 || polls > (1ll << 31)) ? static_cast<long long>(cpn::LOOKBACK_SPIN_LIMIT) : polls;
  return static_cast<int64_t>(cpn::g_spin_limit.exchange(v));
}

int cpn_set_tile_order(int single) { return cpn::g_tile_order.exchange(single != 0 ? 1 : 0); }

int cpn_set_bitonic_rows(int enabled) { return cpn::g_bitonic_rows.exchange(enabled != 0 ? 1 : 0); }

int cpn_set_merge_rows(int mode) { return cpn::g_merge_rows.exchange(mode < 0 ? 1 : mode); }

int64_t cpn_set_wave_row_limit(int64_t limit)
{
  return static_cast<int64_t>(cpn::g_wave_row_limit.exchange(limit < 0 ? 1024ll : static_cast<long long>(limit)));
}

uint64_t cpn_dtype_size(int dtype) { return static_cast<uint64_t>(cpn::key_kind(dtype).bytes); }

uint64_t cpn_key_order_bits(int dtype, uint64_t raw_bits)
{
  const cpn::KeyKind k = cpn::key_kind(dtype);
  if (k.bytes == 0 || k.codec < 0 || k.codec == cpn::CODEC_COMPLEX) {
    return 0;  // complex keys are wider than 64 bits
  }
  switch (k.bytes * 4 + k.codec) {
    case 1 * 4 + cpn::CODEC_UNSIGNED: return cpn::ordered_bits<cpn::CODEC_UNSIGNED, uint8_t>(static_cast<uint8_t>(raw_bits));
    case 1 * 4 + cpn::CODEC_SIGNED: return cpn::ordered_bits<cpn::CODEC_SIGNED, uint8_t>(static_cast<uint8_t>(raw_bits));
    case 2 * 4 + cpn::CODEC_UNSIGNED: return cpn::ordered_bits<cpn::CODEC_UNSIGNED, uint16_t>(static_cast<uint16_t>(raw_bits));
    case 2 * 4 + cpn::CODEC_SIGNED: return cpn::ordered_bits<cpn::CODEC_SIGNED, uint16_t>(static_cast<uint16_t>(raw_bits));
    case 2 * 4 + cpn::CODEC_FLOAT: return cpn::ordered_bits<cpn::CODEC_FLOAT, uint16_t>(static_cast<uint16_t>(raw_bits));
    case 4 * 4 + cpn::CODEC_UNSIGNED: return cpn::ordered_bits<cpn::CODEC_UNSIGNED, uint32_t>(static_cast<uint32_t>(raw_bits));
    case 4 * 4 + cpn::CODEC_SIGNED: return cpn::ordered_bits<cpn::CODEC_SIGNED, uint32_t>(static_cast<uint32_t>(raw_bits));
    case 4 * 4 + cpn::CODEC_FLOAT: return cpn::ordered_bits<cpn::CODEC_FLOAT, uint32_t>(static_cast<uint32_t>(raw_bits));
    case 8 * 4 + cpn::CODEC_UNSIGNED: return cpn::ordered_bits<cpn::CODEC_UNSIGNED, uint64_t>(raw_bits);
    case 8 * 4 + cpn::CODEC_SIGNED: return cpn::ordered_bits<cpn::CODEC_SIGNED, uint64_t>(raw_bits);
    case 8 * 4 + cpn::CODEC_FLOAT: return cpn::ordered_bits<cpn::CODEC_FLOAT, uint64_t>(raw_bits);
    default: return 0;
  }
}

uint64_t cpn_local_sort_temp_bytes(int dtype, uint64_t volume, uint64_t sort_dim_size, int want_values,
                                   int want_indices, int in_place)
{
  const cpn::KeyKind k = cpn::key_kind(dtype);
  if (k.bytes == 0 || k.codec < 0) {
    return 0;
  }
  if (volume == 0) {
    return cpn::HEADER_BYTES;
  }
  if (sort_dim_size == 0 || volume % sort_dim_size != 0) {
    return 0;
  }
  return cpn::workspace_bytes(k.bytes, cpn::key_passes(k.bytes, k.codec), volume, sort_dim_size, want_values != 0, want_indices != 0, in_place != 0);
}

int cpn_local_sort(int dtype, const void* values_in, void* values_out, int64_t* indices_out, uint64_t volume,
                   uint64_t sort_dim_size, int64_t index_offset, int stable, void* temp, uint64_t temp_bytes,
                   void* stream)
{
  return cpn_local_sort_ex(dtype, values_in, values_out, indices_out, volume, sort_dim_size, index_offset, stable, 0u,
                           temp, temp_bytes, stream);
}

int cpn_local_sort_ex(int dtype, const void* values_in, void* values_out, int64_t* indices_out, uint64_t volume,
                      uint64_t sort_dim_size, int64_t index_offset, int stable, uint32_t options, void* temp,
                      uint64_t temp_bytes, void* stream)
{
  (void)stable;  // every path is stable
  if ((options & ~static_cast<uint32_t>(CPN_SORT_SINGLE_TICKET)) != 0) {
    return CPN_ERR_UNSUPPORTED;
  }
  const cpn::KeyKind k = cpn::key_kind(dtype);
  if (k.bytes == 0) {
    return CPN_ERR_DTYPE;
  }
  if (k.codec < 0) {
    return CPN_ERR_UNSUPPORTED;
  }
  if (volume == 0) {
    return CPN_OK;
  }
  if (sort_dim_size == 0 || volume % sort_dim_size != 0) {
    return CPN_ERR_SHAPE;
  }
  if (values_in == nullptr || (values_out == nullptr && indices_out == nullptr)) {
    return CPN_ERR_NULL;
  }
  const uintptr_t kmask = static_cast<uintptr_t>(k.bytes - 1);
  if ((reinterpret_cast<uintptr_t>(values_in) & kmask) != 0 || (reinterpret_cast<uintptr_t>(values_out) & kmask) != 0 ||
      (reinterpret_cast<uintptr_t>(indices_out) & 7u) != 0) {
    return CPN_ERR_ALIGN;
  }
  cpn::SortRequest r{};
  r.values_in    = values_in;
  r.values_out   = values_out;
  r.indices_out  = indices_out;
  r.volume       = volume;
  r.seg          = sort_dim_size;
  r.index_offset = index_offset;
  r.temp         = temp;
  r.temp_bytes   = temp_bytes;
  r.stream       = static_cast<hipStream_t>(stream);
  r.single_ticket = (options & CPN_SORT_SINGLE_TICKET) != 0;
  switch (k.bytes) {
    case 1: return cpn::sort_keys8(k.codec, r);
    case 2: return cpn::sort_keys16(k.codec, r);
    case 4: return cpn::sort_keys32(k.codec, r);
    case 8: return cpn::sort_keys64(k.codec, r);
    case 16: return cpn::sort_keys128(k.codec, r);
    default: return CPN_ERR_UNSUPPORTED;
  }
}

int cpn_local_sort_static(int dtype, const void* values_in, void* values_out, int64_t* indices_out, uint64_t volume,
                          uint64_t sort_dim_size, int64_t index_offset, int stable, uint32_t* status_out, void* stream)
{
  if ((reinterpret_cast<uintptr_t>(status_out) & 3u) != 0) {
    return CPN_ERR_ALIGN;
  }
  const cpn::KeyKind k = cpn::key_kind(dtype);
  if (k.bytes != 0 && k.codec >= 0 && volume != 0 && sort_dim_size != 0 && volume % sort_dim_size == 0) {
    // a well-formed request: does its workspace fit?  (everything else gets cpn_local_sort's own answer)
    const uint64_t need = cpn_local_sort_temp_bytes(dtype, volume, sort_dim_size, values_out != nullptr,
                                                    indices_out != nullptr, values_out == values_in);
    if (need > CPN_STATIC_SCRATCH_BYTES) {
      return CPN_ERR_SCRATCH;
    }
  }
  void* ws = nullptr;
  if (volume != 0) {
    const int rc = cpn::static_scratch_of_current_device(&ws);
    if (rc != CPN_OK) {
      return rc;
    }
  }
  const int rc = cpn_local_sort(dtype, values_in, values_out, indices_out, volume, sort_dim_size, index_offset, stable,
                                ws, CPN_STATIC_SCRATCH_BYTES, stream);
  if (rc != CPN_OK || status_out == nullptr || volume == 0) {
    return rc;
  }
  hipLaunchKernelGGL(cpn::copy_status_kernel, dim3(1), dim3(cpn::WAVE), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint32_t*>(ws), status_out);
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

int cpn_local_sort_check(const void* temp, void* stream)
{
  if (temp == nullptr) {
    return CPN_ERR_NULL;
  }
  uint32_t word = 0;
  CPN_HIP_TRY(hipMemcpyAsync(&word, temp, sizeof(word), hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)));
  CPN_HIP_TRY(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  return word == 0 ? CPN_OK : CPN_ERR_DEVICE;
}

int cpn_swapaxes_copy(int elem_bytes, const void* in, void* out, const int64_t* shape, int ndim, int axis_a, int axis_b,
                      void* stream)
{
  if (shape == nullptr && ndim > 0) {
    return CPN_ERR_NULL;
  }
  if (ndim < 0 || ndim > 8 || (ndim == 0 && (axis_a != 0 || axis_b != 0))) {
    return CPN_ERR_SHAPE;
  }
  if (ndim > 0 && (axis_a < 0 || axis_a >= ndim || axis_b < 0 || axis_b >= ndim)) {
    return CPN_ERR_SHAPE;
  }
  if (elem_bytes != 1 && elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8 && elem_bytes != 16) {
    return CPN_ERR_SHAPE;
  }
  uint64_t total = 1;
  for (int i = 0; i < ndim; ++i) {
    if (shape[i] < 0) {
      return CPN_ERR_SHAPE;
    }
    total *= static_cast<uint64_t>(shape[i]);
  }
  if (total == 0) {
    return CPN_OK;
  }
  if (in == nullptr || out == nullptr) {
    return CPN_ERR_NULL;
  }
  const uintptr_t mask = static_cast<uintptr_t>(elem_bytes - 1);
  if ((reinterpret_cast<uintptr_t>(in) & mask) != 0 || (reinterpret_cast<uintptr_t>(out) & mask) != 0) {
    return CPN_ERR_ALIGN;
  }
  return cpn::swapaxes_copy(elem_bytes, in, out, shape, ndim, axis_a, axis_b, static_cast<hipStream_t>(stream));
}

}  // extern "C"
