// Dense copy with two axes exchanged.  When the second axis is the last one (the only case
// the sort path produces) this is a batched 2-D transpose staged through a padded LDS tile
// so that both the HBM reads and the HBM writes are contiguous along a wavefront.
//
// Replaces the UNARY_OP(COPY) of a transposed store issued by sort_swapped
// (cupynumeric/_thunk/_sort.py:50-76); the reference runs it as one thread per element with
// strided reads (src/cupynumeric/unary/unary_op.cu:85-96,124-170, src/cupynumeric/pitches.h:45-55).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sort_driver.h"

namespace cpn {

// in : [P][A][M][B]   element (p, ia, m, ib)
// out: [P][B][M][A]   element (p, ib, m, ia)
template <typename T, int TS>
__global__ __launch_bounds__(256) void transpose_last_kernel(const T* __restrict__ in,
                                                              T* __restrict__ out,
                                                              uint64_t A,
                                                              uint64_t M,
                                                              uint64_t B,
                                                              uint32_t tiles_a,
                                                              uint32_t tiles_b)
{
  constexpr int ROWS_PER_STEP = 256 / TS;
  __shared__ T tile[TS][TS + 1];

  uint64_t bid        = blockIdx.x;
  const uint32_t tb   = static_cast<uint32_t>(bid % tiles_b);
  bid /= tiles_b;
  const uint32_t ta   = static_cast<uint32_t>(bid % tiles_a);
  const uint64_t batch = bid / tiles_a;
  const uint64_t p    = batch / M;
  const uint64_t m    = batch - p * M;
  const uint64_t in_base  = (p * A * M + m) * B;
  const uint64_t out_base = (p * B * M + m) * A;
  const uint64_t in_row   = M * B;
  const uint64_t out_row  = M * A;

  const int tx = threadIdx.x % TS;
  const int ty = threadIdx.x / TS;
  // A tile that lies inside the array takes the path without bounds checks, in which every load of
  // a thread is issued before the first one is used (under a per-element check the compiler waits
  // for each load before it issues the next).
  const bool inside = (static_cast<uint64_t>(ta) + 1) * TS <= A && (static_cast<uint64_t>(tb) + 1) * TS <= B;
  if (inside) {
    constexpr int STEPS = TS / ROWS_PER_STEP;
    const T* src        = in + in_base + (static_cast<uint64_t>(ta) * TS + ty) * in_row + static_cast<uint64_t>(tb) * TS + tx;
    T v[STEPS];
#pragma unroll
    for (int k = 0; k < STEPS; ++k) {
      v[k] = src[static_cast<uint64_t>(k) * ROWS_PER_STEP * in_row];
    }
#pragma unroll
    for (int k = 0; k < STEPS; ++k) {
      tile[ty + k * ROWS_PER_STEP][tx] = v[k];
    }
    __syncthreads();
    T* dst = out + out_base + (static_cast<uint64_t>(tb) * TS + ty) * out_row + static_cast<uint64_t>(ta) * TS + tx;
#pragma unroll
    for (int k = 0; k < STEPS; ++k) {
      dst[static_cast<uint64_t>(k) * ROWS_PER_STEP * out_row] = tile[tx][ty + k * ROWS_PER_STEP];
    }
    return;
  }
  {
    const uint64_t ib = static_cast<uint64_t>(tb) * TS + tx;
#pragma unroll 4
    for (int r = ty; r < TS; r += ROWS_PER_STEP) {
      const uint64_t ia = static_cast<uint64_t>(ta) * TS + r;
      if (ia < A && ib < B) {
        tile[r][tx] = in[in_base + ia * in_row + ib];
      }
    }
  }
  __syncthreads();
  {
    const uint64_t ia = static_cast<uint64_t>(ta) * TS + tx;
#pragma unroll 4
    for (int r = ty; r < TS; r += ROWS_PER_STEP) {
      const uint64_t ib = static_cast<uint64_t>(tb) * TS + r;
      if (ia < A && ib < B) {
        out[out_base + ib * out_row + ia] = tile[tx][r];
      }
    }
  }
}

// 2-byte elements, both extents even and both pointers 4-byte aligned: 128 x 128 tiles moved as
// 32-bit words.  A thread loads the two words of a 2 x 2 block, exchanges the halves in
// registers (v_perm_b32) and stores two words that already hold two elements of an output
// row each, so that the LDS tile is transposed at word granularity and every HBM access of a
// wavefront is 256 contiguous bytes.
constexpr int PAIR_TS = 128;
__global__ __launch_bounds__(256) void transpose_pairs_kernel(const uint32_t* __restrict__ in,
                                                               uint32_t* __restrict__ out,
                                                               uint64_t A,
                                                               uint64_t M,
                                                               uint64_t B,
                                                               uint32_t tiles_a,
                                                               uint32_t tiles_b)
{
  constexpr int HP = PAIR_TS / 2;  // words per tile row
  __shared__ uint32_t tile[PAIR_TS][HP + 1];  // [column of the input][pair of input rows]

  uint64_t bid         = blockIdx.x;
  const uint32_t tb    = static_cast<uint32_t>(bid % tiles_b);
  bid /= tiles_b;
  const uint32_t ta    = static_cast<uint32_t>(bid % tiles_a);
  const uint64_t batch = bid / tiles_a;
  const uint64_t p     = batch / M;
  const uint64_t m     = batch - p * M;
  // element offsets; all even, so halving them gives word offsets
  const uint64_t in_base  = (p * A * M + m) * B;
  const uint64_t out_base = (p * B * M + m) * A;
  const uint64_t in_row   = M * B;
  const uint64_t out_row  = M * A;
  const uint64_t a0       = static_cast<uint64_t>(ta) * PAIR_TS;
  const uint64_t b0       = static_cast<uint64_t>(tb) * PAIR_TS;

  const int x = threadIdx.x % HP;  // word inside a row (load: column pair, store: row pair)
  const int y = threadIdx.x / HP;  // 0..3
  // (tiles inside the array: no bounds checks, every load of a thread issued before the first use)
  if (a0 + PAIR_TS <= A && b0 + PAIR_TS <= B) {
    constexpr int YS    = 256 / HP;      // row pairs in flight per step
    constexpr int STEPS = HP / YS;       // 16
    const uint32_t* src = in + (in_base + (a0 + 2 * y) * in_row + b0 + 2 * x) / 2;
    const uint64_t pair_stride = (2 * YS * in_row) / 2;  // words between the row pairs of two steps
    const uint64_t row_words   = in_row / 2;
    uint32_t w0[STEPS], w1[STEPS];
#pragma unroll
    for (int k = 0; k < STEPS; ++k) {
      w0[k] = src[k * pair_stride];
      w1[k] = src[k * pair_stride + row_words];
    }
#pragma unroll
    for (int k = 0; k < STEPS; ++k) {
      const int rp        = y + k * YS;
      tile[2 * x][rp]     = __builtin_amdgcn_perm(w1[k], w0[k], 0x05040100u);
      tile[2 * x + 1][rp] = __builtin_amdgcn_perm(w1[k], w0[k], 0x07060302u);
    }
    __syncthreads();
    uint32_t* dst = out + (out_base + (b0 + y) * out_row + a0 + 2 * x) / 2;
    const uint64_t out_step = (YS * out_row) / 2;
#pragma unroll
    for (int k = 0; k < PAIR_TS / YS; ++k) {
      dst[k * out_step] = tile[y + k * YS][x];
    }
    return;
  }
  {
    const uint64_t ib = b0 + 2 * x;
#pragma unroll 4
    for (int rp = y; rp < HP; rp += 256 / HP) {
      const uint64_t ia = a0 + 2 * rp;
      if (ia < A && ib < B) {
        const uint32_t w0 = in[(in_base + ia * in_row + ib) / 2];        // x[ia][ib], x[ia][ib+1]
        const uint32_t w1 = in[(in_base + (ia + 1) * in_row + ib) / 2];  // x[ia+1][ib], x[ia+1][ib+1]
        tile[2 * x][rp]     = __builtin_amdgcn_perm(w1, w0, 0x05040100u);  // x[ia][ib],   x[ia+1][ib]
        tile[2 * x + 1][rp] = __builtin_amdgcn_perm(w1, w0, 0x07060302u);  // x[ia][ib+1], x[ia+1][ib+1]
      }
    }
  }
  __syncthreads();
  {
    const uint64_t ia = a0 + 2 * x;
#pragma unroll 4
    for (int c = y; c < PAIR_TS; c += 256 / HP) {
      const uint64_t ib = b0 + c;
      if (ia < A && ib < B) {
        out[(out_base + ib * out_row + ia) / 2] = tile[c][x];
      }
    }
  }
}

// General case: in [P][A][M][B][Q] -> out [P][B][M][A][Q], one output element per thread step.
template <typename T>
__global__ __launch_bounds__(256) void swapaxes_generic_kernel(const T* __restrict__ in,
                                                                T* __restrict__ out,
                                                                uint64_t A,
                                                                uint64_t M,
                                                                uint64_t B,
                                                                uint64_t Q,
                                                                uint64_t total)
{
  const uint64_t stride = static_cast<uint64_t>(gridDim.x) * blockDim.x;
  for (uint64_t o = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; o < total; o += stride) {
    uint64_t t        = o;
    const uint64_t q  = t % Q;
    t /= Q;
    const uint64_t ia = t % A;
    t /= A;
    const uint64_t m  = t % M;
    t /= M;
    const uint64_t ib = t % B;
    const uint64_t p  = t / B;
    out[o]            = in[(((p * A + ia) * M + m) * B + ib) * Q + q];
  }
}

template <typename T, int TS>
static int swapaxes_typed(const void* in, void* out, uint64_t P, uint64_t A, uint64_t M, uint64_t B, uint64_t Q,
                          hipStream_t stream)
{
  const uint64_t total = P * A * M * B * Q;
  if constexpr (sizeof(T) == 2) {
    if (Q == 1 && A % 2 == 0 && B % 2 == 0 && (reinterpret_cast<uintptr_t>(in) % 4) == 0 &&
        (reinterpret_cast<uintptr_t>(out) % 4) == 0) {
      const uint64_t tiles_a = (A + PAIR_TS - 1) / PAIR_TS;
      const uint64_t tiles_b = (B + PAIR_TS - 1) / PAIR_TS;
      const uint64_t grid    = tiles_a * tiles_b * P * M;
      if (tiles_a < (1ull << 31) && tiles_b < (1ull << 31) && grid < (1ull << 31)) {
        {
          ProfileScope prof("transpose_last", stream);
          hipLaunchKernelGGL(transpose_pairs_kernel, dim3(static_cast<uint32_t>(grid)), dim3(256), 0, stream,
                             static_cast<const uint32_t*>(in), static_cast<uint32_t*>(out), A, M, B,
                             static_cast<uint32_t>(tiles_a), static_cast<uint32_t>(tiles_b));
        }
        CPN_HIP_TRY(hipGetLastError());
        return CPN_OK;
      }
    }
  }
  if (Q == 1) {
    const uint64_t tiles_a = (A + TS - 1) / TS;
    const uint64_t tiles_b = (B + TS - 1) / TS;
    const uint64_t grid    = tiles_a * tiles_b * P * M;
    if (tiles_a >= (1ull << 31) || tiles_b >= (1ull << 31) || grid >= (1ull << 31)) {
      return CPN_ERR_UNSUPPORTED;
    }
    ProfileScope prof("transpose_last", stream);
    hipLaunchKernelGGL((transpose_last_kernel<T, TS>), dim3(static_cast<uint32_t>(grid)), dim3(256), 0, stream,
                       static_cast<const T*>(in), static_cast<T*>(out), A, M, B, static_cast<uint32_t>(tiles_a),
                       static_cast<uint32_t>(tiles_b));
  } else {
    uint64_t grid = (total + 255) / 256;
    if (grid > 65536) {
      grid = 65536;
    }
    ProfileScope prof("swapaxes_generic", stream);
    hipLaunchKernelGGL((swapaxes_generic_kernel<T>), dim3(static_cast<uint32_t>(grid)), dim3(256), 0, stream,
                       static_cast<const T*>(in), static_cast<T*>(out), A, M, B, Q, total);
  }
  CPN_HIP_TRY(hipGetLastError());
  return CPN_OK;
}

int swapaxes_copy(int elem_bytes, const void* in, void* out, const int64_t* shape, int ndim, int axis_a, int axis_b,
                  hipStream_t stream)
{
  if (axis_a > axis_b) {
    const int t = axis_a;
    axis_a      = axis_b;
    axis_b      = t;
  }
  uint64_t P = 1, A = 1, M = 1, B = 1, Q = 1;
  for (int i = 0; i < ndim; ++i) {
    const uint64_t e = static_cast<uint64_t>(shape[i]);
    if (i < axis_a) {
      P *= e;
    } else if (i == axis_a) {
      A = e;
    } else if (i < axis_b) {
      M *= e;
    } else if (i == axis_b) {
      B = e;
    } else {
      Q *= e;
    }
  }
  if (axis_a == axis_b) {
    B = 1;  // shape[axis] was assigned to A; nothing moves
  }
  const uint64_t total = P * A * M * B * Q;
  if (total == 0) {
    return CPN_OK;
  }
  // exchanging with (or across only) unit axes leaves the memory order unchanged
  const bool identity = (axis_a == axis_b) || (A == 1 && B == 1) || (M == 1 && (A == 1 || B == 1));
  if (identity) {
    CPN_HIP_TRY(hipMemcpyAsync(out, in, total * elem_bytes, hipMemcpyDeviceToDevice, stream));
    return CPN_OK;
  }
  switch (elem_bytes) {
    case 1: return swapaxes_typed<uint8_t, 64>(in, out, P, A, M, B, Q, stream);
    case 2: return swapaxes_typed<uint16_t, 64>(in, out, P, A, M, B, Q, stream);
    case 4: return swapaxes_typed<uint32_t, 64>(in, out, P, A, M, B, Q, stream);
    case 8: return swapaxes_typed<uint64_t, 64>(in, out, P, A, M, B, Q, stream);
    case 16: return swapaxes_typed<uint4, 32>(in, out, P, A, M, B, Q, stream);
    default: return CPN_ERR_SHAPE;
  }
}

}  // namespace cpn
