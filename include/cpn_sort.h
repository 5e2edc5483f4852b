/*
 * cpn_sort.h -- C ABI of the MI355X (gfx950) sort / argsort library `libcpnsort.so`.
 *
 * The library replaces the single-processor GPU sort of cuPyNumeric's SORT task.  In the
 * reference that work sits behind typed, plain pointer+size functions
 *
 *   local_sort<CODE>(const VAL* values_in, VAL* values_out, const int64_t* indices_in,
 *                    int64_t* indices_out, size_t volume, size_t sort_dim_size,
 *                    bool stable, cudaStream_t)            src/cupynumeric/sort/sort.cu:63-96
 *   cub_local_sort(...)   x12 dtypes                        src/cupynumeric/sort/cub_sort.h:21-115
 *   thrust_local_sort(...) x14 dtypes                       src/cupynumeric/sort/thrust_sort.h:21-145
 *
 * which SortImplBody<GPU> (src/cupynumeric/sort/sort.cu:1797-1940) calls after it has picked
 * the output/temporary buffers.  The entry points below are what a binding for that call
 * site links against.  Everything is `extern "C"`, takes raw device pointers, sizes and a
 * `hipStream_t` passed as `void*`; no C++ or torch types cross the boundary.
 *
 * All functions are asynchronous with respect to the host unless stated otherwise, never
 * abort the process and never free caller memory.  They return CPN_OK (0) or a negative
 * cpn_status.  The caller owns every buffer, including the temporary workspace.
 */
#ifndef CPN_SORT_H
#define CPN_SORT_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Element type codes.  Order follows the per-dtype instantiation list of the reference
 * (src/cupynumeric/sort/cub_sort.h:21-115, thrust_sort.h:129-145). */
typedef enum cpn_dtype {
  CPN_BOOL       = 0,
  CPN_INT8       = 1,
  CPN_INT16      = 2,
  CPN_INT32      = 3,
  CPN_INT64      = 4,
  CPN_UINT8      = 5,
  CPN_UINT16     = 6,
  CPN_UINT32     = 7,
  CPN_UINT64     = 8,
  CPN_FLOAT16    = 9,
  CPN_FLOAT32    = 10,
  CPN_FLOAT64    = 11,
  CPN_COMPLEX64  = 12,
  CPN_COMPLEX128 = 13
} cpn_dtype;

typedef enum cpn_status {
  CPN_OK              = 0,
  CPN_ERR_DTYPE       = -1, /* unknown or unsupported element type code              */
  CPN_ERR_NULL        = -2, /* a required pointer is NULL                              */
  CPN_ERR_SHAPE       = -3, /* sort_dim_size is 0 or does not divide volume, bad axes  */
  CPN_ERR_TEMP        = -4, /* workspace missing, too small or not 256-byte aligned    */
  CPN_ERR_ALIGN       = -5, /* a data pointer is not aligned to its element size       */
  CPN_ERR_HIP         = -6, /* a HIP runtime call failed (see cpn_last_hip_error)      */
  CPN_ERR_DEVICE      = -7, /* a kernel flagged an internal failure (bounded wait hit) */
  CPN_ERR_UNSUPPORTED = -8, /* valid request that this build does not implement        */
  CPN_ERR_SCRATCH     = -9  /* cpn_local_sort_static: the request needs more workspace
                               than CPN_STATIC_SCRATCH_BYTES                            */
} cpn_status;

/* Library version, (major << 16) | minor. */
int cpn_sort_version(void);

/* Static, human readable text for a cpn_status value. */
const char* cpn_status_string(int status);

/* hipError_t of the last HIP call that failed on the calling thread (0 if none). */
int cpn_last_hip_error(void);

/* Size in bytes of one element of `dtype`, or 0 for an unknown code. */
uint64_t cpn_dtype_size(int dtype);

/*
 * Host-side image of the key transform the kernels apply before extracting radix digits:
 * the unsigned integer (of the element's width) whose natural order is the sort order of
 * the element with raw bit pattern `raw_bits`.  Pure host arithmetic, for tests and
 * debugging.  Stands where the reference relies on cub's radix key traits
 * (src/cupynumeric/sort/cub_sort.cuh:60-71); unlike those it maps every NaN to the maximum
 * and -0.0 to the key of +0.0.  Returns 0 for unknown or unsupported codes.
 */
uint64_t cpn_key_order_bits(int dtype, uint64_t raw_bits);

/*
 * Workspace size, in bytes, that cpn_local_sort needs for this request.  Pure host
 * arithmetic (no HIP call); returns 0 when the request itself is invalid.  Replaces the
 * size query of cub::DeviceRadixSort (src/cupynumeric/sort/cub_sort.cuh:56-63).
 *
 *   want_values  != 0  sorted values are written (values_out != NULL)
 *   want_indices != 0  int64 indices are written (indices_out != NULL)
 *   in_place     != 0  values_out aliases values_in
 */
uint64_t cpn_local_sort_temp_bytes(int dtype, uint64_t volume, uint64_t sort_dim_size,
                                   int want_values, int want_indices, int in_place);

/*
 * Stable sort of `volume / sort_dim_size` independent rows of `sort_dim_size` elements,
 * dense row-major.  Replaces local_sort<CODE> (src/cupynumeric/sort/sort.cu:63-96) together
 * with the index initialisation that precedes it (sort.cu:1851-1863, sort.h:83-92).
 *
 *   values_in    device pointer, read only unless it equals values_out
 *   values_out   sorted values (same element type), may equal values_in; NULL when only
 *                indices are wanted
 *   indices_out  int64 position of every sorted element inside its row plus index_offset
 *                (the reference's `i % sort_dim_size + offset`); NULL for a plain sort
 *   stable       accepted for signature parity; the result is always stable, which
 *                satisfies both settings
 *   temp         workspace of at least cpn_local_sort_temp_bytes(...) bytes, 256-byte
 *                aligned; its contents are undefined afterwards
 *   stream       hipStream_t (NULL = the null stream)
 *
 * Ordering is NumPy's: integers by value, bool false < true, floating point ascending with
 * every NaN after +inf, and -0.0 equal to +0.0 (ties keep input order).  Bit patterns of
 * the elements are moved unchanged.  volume == 0 is a successful no-op.
 */
int cpn_local_sort(int dtype, const void* values_in, void* values_out, int64_t* indices_out,
                   uint64_t volume, uint64_t sort_dim_size, int64_t index_offset, int stable,
                   void* temp, uint64_t temp_bytes, void* stream);

/*
 * cpn_local_sort with per-call options (a bit set of CPN_SORT_*; 0 = cpn_local_sort; unknown bits
 * return CPN_ERR_UNSUPPORTED).  Same call site as cpn_local_sort (src/cupynumeric/sort/sort.cu:63-96);
 * the options have no counterpart in the reference.
 *
 *   CPN_SORT_SINGLE_TICKET  the scatter passes of this call hand their tiles to workgroups through
 *                           one counter for the whole launch instead of one per XCD.  Slower by a few
 *                           per cent, and independent of every XCD of the device taking part in the
 *                           launch: the way to repeat a sort that came back with CPN_ERR_DEVICE
 *                           (cpn_local_sort_check), without touching process-wide state.  Results do
 *                           not depend on it.
 */
#define CPN_SORT_SINGLE_TICKET 1u
int cpn_local_sort_ex(int dtype, const void* values_in, void* values_out, int64_t* indices_out,
                      uint64_t volume, uint64_t sort_dim_size, int64_t index_offset, int stable,
                      uint32_t options, void* temp, uint64_t temp_bytes, void* stream);

/*
 * cpn_local_sort for callers that cannot allocate device memory or pass a workspace: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference, whose sort always draws its temporaries from a Legate pool
 * (src/cupynumeric/sort/cub_sort.cuh:48,62-63).
 *
 * Same arguments, results and ordering as cpn_local_sort, without `temp`: the workspace is a
 * static array of CPN_STATIC_SCRATCH_BYTES bytes of device memory inside the library, one copy
 * per GPU, held until the process ends.  The call allocates and frees nothing (no hipMalloc,
 * hipFree or allocating library routine) and launches the same kernels as cpn_local_sort.
 *
 *   - a request whose cpn_local_sort_temp_bytes exceeds CPN_STATIC_SCRATCH_BYTES returns
 *     CPN_ERR_SCRATCH and launches nothing (row sorts that fit the per-row kernels need 2 KiB
 *     whatever their volume; a 1-D argsort of 4-byte keys fits up to about 5.4 million keys);
 *   - status_out (device memory, 4-byte aligned, may be NULL) receives the sort's device status
 *     word when the sort has finished: 0, or non-zero when a bounded wait inside a kernel ran out
 *     and the output is invalid (what cpn_local_sort_check reports for cpn_local_sort);
 *   - every call on one GPU uses that GPU's one array, whatever its stream: calls that overlap in
 *     time on one GPU race.  Order them on one stream, or with events;
 *   - the first call on a device is the set-up: it looks up the array's address on that device
 *     (hipGetSymbolAddress), and the HIP runtime brings the array into device memory with the
 *     library's code then; make that call outside graph capture and before the part of the
 *     program that must not allocate.
 */
#define CPN_STATIC_SCRATCH_BYTES (64ull << 20)
int cpn_local_sort_static(int dtype, const void* values_in, void* values_out, int64_t* indices_out,
                          uint64_t volume, uint64_t sort_dim_size, int64_t index_offset, int stable,
                          uint32_t* status_out, void* stream);

/*
 * Blocks until `stream` has finished, then reports what the kernels of the last
 * cpn_local_sort call that used `temp` recorded in its status word: CPN_OK, or
 * CPN_ERR_DEVICE when a bounded wait inside a kernel ran out (the output is then invalid).
 * The reference has no counterpart: device failures abort the process there
 * (src/cupynumeric/cuda_help.h:167-180).
 */
int cpn_local_sort_check(const void* temp, void* stream);

/*
 * out = in with axes `axis_a` and `axis_b` exchanged, both dense row-major; `shape` is the
 * shape of `in`.  Replaces the UNARY_OP(COPY) of a transposed store that sort_swapped
 * issues (cupynumeric/_thunk/_sort.py:50-76, src/cupynumeric/unary/unary_op.cu:85-96,124-170).
 * elem_bytes is 1, 2, 4, 8 or 16; ndim <= 8; in and out must not overlap.
 */
int cpn_swapaxes_copy(int elem_bytes, const void* in, void* out, const int64_t* shape, int ndim,
                      int axis_a, int axis_b, void* stream);

/*
 * out[i] = complex(in[i], 0): `in` holds `volume` elements of the real type `src_dtype`, `out`
 * receives complex64 or complex128 (`dst_dtype`).  The cast sort_complex applies to real
 * results (cupynumeric/_module/ssc_sorting.py:150-159: `result.astype(np.complex64 / complex128)`).
 */
int cpn_real_to_complex(int src_dtype, const void* in, int dst_dtype, void* out, uint64_t volume,
                        void* stream);

/*
 * out[i] = (dst type) in[i] for `volume` elements; any of the 14 element types to any other.
 * Conversions follow C++ static_cast (float16 goes through float32), bool results are
 * `x != 0`, complex -> real keeps the real part.  Used for the `astype` to the common type
 * that searchsorted applies to its two arguments (cupynumeric/_array/array.py:3743-3751); a
 * UNARY_OP convert task in the reference (src/cupynumeric/unary/convert.cu).
 */
int cpn_astype(int src_dtype, const void* in, int dst_dtype, void* out, uint64_t volume, void* stream);

/*
 * positions_out[i] = where values[i] would be inserted into the ascending array `sorted` of n
 * elements: the first position whose element is not less than the value (left != 0, NumPy
 * side='left') or the first position whose element is greater (left == 0, side='right').
 * Both arrays have element type `dtype`; the order is the one cpn_local_sort produces.
 * Replaces SearchSortedTask::gpu_variant (src/cupynumeric/sort/searchsorted.cu:27-116,
 * cupynumeric/_thunk/deferred.py:5425-5451) for a sorted array held by one GPU.
 *
 * `temp` is optional.  cpn_searchsorted_temp_bytes returns the size of the workspace with
 * which a large search (sorted array beyond the caches, many values) first sorts the values
 * so that neighbouring lanes probe neighbouring memory, or 0 when the request is searched
 * directly anyway.  With temp == NULL, or a workspace smaller than that, the values are
 * searched in the order given; the results are the same.  A workspace must be 256-byte
 * aligned; when it is used its first word is the sort's device status
 * (cpn_local_sort_check applies).
 */
uint64_t cpn_searchsorted_temp_bytes(int dtype, uint64_t n, uint64_t num_values);
int cpn_searchsorted(int dtype, const void* sorted, uint64_t n, const void* values,
                     uint64_t num_values, int left, int64_t* positions_out, void* temp,
                     uint64_t temp_bytes, void* stream);

/*
 * Sorted distinct values.  values_out has room for `volume` elements and receives the
 * distinct values in ascending order (the first of every run of equal keys in the stable
 * sorted order: all NaNs count as one value, -0.0 and +0.0 as one); *count_out (device
 * memory, 8-byte aligned) receives how many there are.  `temp` is a 256-byte aligned
 * workspace of at least cpn_unique_temp_bytes(dtype, volume) bytes; the device status word of
 * the sort is at its start, so cpn_local_sort_check(temp, stream) applies.  values_in is not
 * modified.  Replaces UniqueTask::gpu_variant on one processor
 * (src/cupynumeric/set/unique.cu:137-204, cupynumeric/_thunk/deferred.py:5375-5395).
 * cpn_unique_temp_bytes returns 0 for an unknown dtype.
 */
uint64_t cpn_unique_temp_bytes(int dtype, uint64_t volume);
int cpn_unique(int dtype, const void* values_in, void* values_out, uint64_t volume,
               uint64_t* count_out, void* temp, uint64_t temp_bytes, void* stream);

/*
 * Quantiles along the middle axis of `sorted`, a dense [outer][n][inner] array that is already
 * sorted along that axis, for num_q quantiles whose positions the caller has worked out:
 *   interpolate == 0   out[q][o][i] = sorted[o][left[q]][i]                       (element type `dtype`)
 *   interpolate != 0   out[q][o][i] = (1 - gamma[q]) * sorted[o][left[q]][i]
 *                                     + gamma[q] * sorted[o][right[q]][i]          (float64)
 * with the two products and the sum rounded separately in the arithmetic the reference's
 * expression has (the element type for float16 / float32 / float64, float64 for integers and bool).
 * left, right (int64, in [0, n)) and gamma (float64) are device arrays of num_q entries; right and
 * gamma may be NULL when interpolate == 0.  Complex types return CPN_ERR_DTYPE.  Replaces the
 * per-quantile take / multiply / add tasks at the end of _quantile_impl
 * (cupynumeric/_module/stats_order.py:249-337), which quantile, percentile and median run after
 * their sort (stats_order.py:476-482, cupynumeric/_module/stats_avgs_vars.py:373-443).
 */
int cpn_quantile_sorted(int dtype, const void* sorted, uint64_t outer, uint64_t n, uint64_t inner,
                        uint64_t num_q, const int64_t* left, const int64_t* right, const double* gamma,
                        int interpolate, void* out, void* stream);

/*
 * The quantiles of nanquantile / nanpercentile / nanmedian, which ignore NaNs
 * (cupynumeric/_module/stats_order.py:653-951, cupynumeric/_module/stats_avgs_vars.py:445-512).
 * `sorted` is a dense [outer][n][inner] array of float16 / float32 / float64 sorted along the middle
 * axis in NumPy order, i.e. with the NaNs of every slice at its end.
 *
 * cpn_count_not_nan_sorted: counts[o][i] (int64) = number of elements of slice (o, i) that are not
 * NaN, by binary search; replaces count_nonzero(logical_not(isnan(a)), axis) (stats_order.py:879-881).
 *
 * cpn_nanquantile_sorted: for quantile q and slice s = (o, i), with left, right (int64) and gamma
 * (float64) device arrays of num_q * outer * inner entries ([q][o][i]) that the caller has worked
 * out from counts[s] (stats_order.py:713-746):
 *   counts[s] == 0      out[q][s] = NaN
 *   interpolate == 0    out[q][s] = v(left[q][s])
 *   interpolate != 0    g = gamma[q][s] rounded to the element type; out[q][s] =
 *                       (1 - g) * v(left[q][s]) + g * v(right[q][s]), every operation rounded in the
 *                       element type, as the reference evaluates it on arrays of that type (:748-757)
 * where v(p) is element p of the slice as the reference sees it: it replaces the NaNs by the largest
 * finite value of the type BEFORE it sorts (:886-887), so in a slice that holds m NaNs the m
 * positions after its last finite element read as that value and +inf elements follow them.
 * `out` holds elements of `dtype` when keep_dtype != 0 (the methods that pick samples, and
 * inverted_cdf), float64 otherwise.  Other dtypes return CPN_ERR_DTYPE.
 */
int cpn_count_not_nan_sorted(int dtype, const void* sorted, uint64_t outer, uint64_t n, uint64_t inner,
                             int64_t* counts, void* stream);
int cpn_nanquantile_sorted(int dtype, const void* sorted, uint64_t outer, uint64_t n, uint64_t inner,
                           uint64_t num_q, const int64_t* counts, const int64_t* left, const int64_t* right,
                           const double* gamma, int interpolate, int keep_dtype, void* out, void* stream);

/*
 * out[r][j] = src[r][indices[r][j]] for `rows` dense rows: src rows hold src_seg elements of
 * elem_bytes (1, 2, 4, 8 or 16) bytes, indices and out rows hold idx_seg elements.  Indices are
 * int64, negative ones count from the end of the row.  An index outside [-src_seg, src_seg)
 * writes nothing and stores 1 to *oob_flag (device memory, may be NULL; the caller clears it).
 * This is the take_along_axis that lexsort applies between its argsorts
 * (cupynumeric/_module/ssc_sorting.py:430-442, cupynumeric/_module/indexing.py:648-760), on the
 * last axis; other axes go through cpn_swapaxes_copy first.  out must not overlap the inputs.
 */
int cpn_take_along_last_axis(int elem_bytes, const void* src, const int64_t* indices, void* out,
                             uint64_t rows, uint64_t src_seg, uint64_t idx_seg, uint32_t* oob_flag,
                             void* stream);

/*
 * cpn_take_along_last_axis when the leading dimensions of `src` and `indices` broadcast against each
 * other (every dimension but the axis may be 1 on either side, cupynumeric/_module/indexing.py:700-760,
 * where the reference falls back to a gather over coordinate arrays).  The output has lead_ndim (0..7)
 * leading dimensions out_lead_shape[] and rows of idx_seg elements; src_lead_strides[d] and
 * idx_lead_strides[d] say how many rows of `src` / `indices` one step in leading dimension d is worth:
 * the dense stride of that side, or 0 where its extent is 1.  Everything else as above.
 */
int cpn_take_along_last_axis_broadcast(int elem_bytes, const void* src, const int64_t* indices, void* out,
                                       int lead_ndim, const uint64_t* out_lead_shape,
                                       const uint64_t* src_lead_strides, const uint64_t* idx_lead_strides,
                                       uint64_t src_seg, uint64_t idx_seg, uint32_t* oob_flag, void* stream);

/*
 * Packs num_keys (1..8) real keys of `rows` dense rows of `seg` elements into one unsigned
 * word per element (packed_bytes = 4 or 8, at least the summed width of the keys):
 * keys[0] is the least significant key, as in lexsort; each key enters as the
 * order-preserving unsigned image of its element type, so that the unsigned order of the
 * packed words is the lexicographic order of the keys under NumPy's rules.  With `indices`
 * (int64, row relative, may be NULL) element j of a row takes its keys from position
 * indices[j] of that row.  An argsort of the packed words (dtype CPN_UINT32 / CPN_UINT64)
 * then replaces the reference's argsort + take_along_axis per key
 * (cupynumeric/_module/ssc_sorting.py:423-444).  Complex keys return CPN_ERR_DTYPE.
 */
int cpn_lexsort_pack(int num_keys, const int* dtypes, const void* const* keys, const int64_t* indices,
                     int packed_bytes, void* packed_out, uint64_t rows, uint64_t seg, void* stream);

/* =============================================================================================
 * Test, A/B and benchmark hooks.  A binding of the reference's call site needs nothing below this
 * line: the entry points above are the product.  The cpn_set_* functions change process-wide
 * state; they exist so that tests can reach kernels that small inputs would not (64-bit row
 * positions, virtual digits, the bounded wait that gives up) and so that benchmarks can compare
 * one kernel with another on the same input.  Call them at start-up or from one thread while no
 * other thread sorts; never from code that serves requests.  Two of them (cpn_set_lds_row_limit,
 * cpn_set_merge_rows) and the two thresholds change what cpn_local_sort_temp_bytes returns:
 * cpn_local_sort works the size out again from the settings in force when it is called and
 * returns CPN_ERR_TEMP, before it launches anything, when the workspace it was given is smaller
 * than that.  Per-call choices go through cpn_local_sort_ex instead.
 * ============================================================================================= */

/*
 * Process-wide tunable: rows of at most `limit` elements are sorted by the one-workgroup-
 * per-row LDS kernel, longer rows by the global radix sort.  Values above the kernel's
 * capacity are clamped to it, a negative value restores the default; the previous setting is
 * returned (-1 = default).  Also initialised from the environment variable
 * CPN_SORT_LDS_ROW_LIMIT.  Plays the role of the reference's compile-time
 * SEGMENT_THRESHOLD_RADIX_SORT (src/cupynumeric/sort/sort.cu:41).  Sizes returned by
 * cpn_local_sort_temp_bytes depend on it: do not change it between the size query and the sort.
 */
int64_t cpn_set_lds_row_limit(int64_t limit);

/*
 * Process-wide tunable: rows of at most `limit` elements (at most 1024) are sorted by one
 * wavefront each, longer rows that fit in LDS by one workgroup each.  A negative value
 * restores the default; the previous setting is returned.  Also initialised from the
 * environment variable CPN_SORT_WAVE_ROW_LIMIT.  Does not affect workspace sizes.
 */
int64_t cpn_set_wave_row_limit(int64_t limit);

/*
 * Process-wide switch: short rows of real keys of up to 8 bytes (2 ... 128 keys; up to 256 keys of 1 byte when
 * positions are returned and of 8 bytes when only values are, 384 for float64; up to 1024 keys of 2 and 4 bytes) are sorted by a
 * network of compare-exchanges on eight to fourteen keys per lane of a wavefront (enabled != 0, the default) or by
 * the ranking kernels that take the other key types of that length (0).  Returns the previous setting.  Also
 * initialised from the environment variable CPN_SORT_BITONIC_ROWS (0 switches it off);
 * CPN_SORT_BITONIC_ROW_LIMIT lowers the longest row that the network takes.  Does not affect workspace sizes.
 * An A/B switch with no counterpart in the reference, which merge-sorts (segment id, value) tuples
 * for short rows (src/cupynumeric/sort/thrust_sort.cuh:68-122).
 */
int cpn_set_bitonic_rows(int enabled);

/*
 * Process-wide switch: rows longer than the per-row kernels take (real keys of 4 and 8 bytes) are cut
 * into 2, 4, ... pieces that the per-row kernel sorts and that are then merged pairwise, level by
 * level, as long as that is cheaper than the global path's one pass per key byte (mode 1, the default:
 * up to 6 levels for 8-byte keys, 5 with positions, i.e. rows of up to 1 048 576 and 458 752 keys;
 * 2 levels for 4-byte keys, rows of up to 65 536), or all go down the global path (mode 0).  A mode N >= 2 allows up to N - 1 levels for every key (A/B runs); a
 * negative mode restores the default.  Returns the previous mode.  Also initialised from the
 * environment variable CPN_SORT_MERGE_ROWS.  Changes the sizes returned by
 * cpn_local_sort_temp_bytes: do not change it between the size query and the sort.
 * An A/B switch with no counterpart in the reference, whose segmented radix sort takes every row
 * length (src/cupynumeric/sort/cub_sort.cuh:81-105).
 */
int cpn_set_merge_rows(int mode);

/*
 * Process-wide tunable: rows of at least `elements` elements on the global path keep their
 * per-row counts, tile descriptors and row positions in 64 bits.  The default and the maximum
 * is 2^30 (shorter rows use 32 bits); a negative value restores the default and the previous
 * setting is returned (-1 = default).  Lower values exist so that tests can run the 64-bit
 * kernels on small inputs; they change workspace sizes (cpn_local_sort_temp_bytes follows).
 * Also initialised from the environment variable CPN_SORT_WIDE_ROW_THRESHOLD.
 */
int64_t cpn_set_wide_row_threshold(int64_t elements);

/*
 * Process-wide tunable: how many times a tile of the global path polls the descriptor of a
 * predecessor before it gives up, sets the device status word (CPN_ERR_DEVICE from
 * cpn_local_sort_check) and lets every kernel run to its end with invalid output.  The default
 * (2^22 polls, restored by a value below 1) is far above any real wait; tests of the failure
 * path set 1.  The previous setting is returned.
 */
int64_t cpn_set_lookback_spin_limit(int64_t polls);

/*
 * Process-wide tunable: how the scatter passes of the global sort hand their tiles to workgroups.
 * 0 (default): per XCD, so that neighbouring tiles share an L2 (faster; assumes that every XCD of
 * the device keeps receiving workgroups of the launch: if foreign work held one XCD for seconds,
 * the bounded look-back would give up with CPN_ERR_DEVICE).  Non-zero: one ticket counter for the
 * whole launch, which has no such dependence (one call at a time: CPN_SORT_SINGLE_TICKET of
 * cpn_local_sort_ex).  Results do not depend on it.  Returns the previous setting.  Also initialised from the
 * environment variable CPN_SORT_TILE_ORDER ("single" selects the one counter).  The reference has no
 * counterpart (cub's onesweep takes tiles from one counter, behind src/cupynumeric/sort/cub_sort.cuh:120-143).
 */
int cpn_set_tile_order(int single);

/*
 * Process-wide tunable: a 1-D sort of real 8-byte keys with at least `elements` elements lets
 * the device replace its eight byte passes by one pass on the ranks of the keys when the row
 * holds at most 256 different keys, or by fewer passes on "virtual digits" when the
 * histograms show that the bytes of the keys take few distinct values (several bytes then
 * share one 8-bit digit; cupynumeric_amd/csrc/virtual_digits.h).  Results do not depend on
 * it.  The default is 2^26 (below that the extra launches outweigh the average gain); a
 * negative value restores it and the previous setting is returned.  It changes workspace
 * sizes by 24 KiB (cpn_local_sort_temp_bytes follows).  Also initialised from the
 * environment variable CPN_SORT_VIRTUAL_DIGIT_THRESHOLD.
 */
int64_t cpn_set_virtual_digit_threshold(int64_t elements);

/*
 * Per-launch timing.  cpn_profile_enable(1) makes every kernel launch of the library record
 * a pair of HIP events on the stream it is launched on; it returns the previous setting.
 * cpn_profile_collect waits for the recorded events, writes up to `max_records` entries --
 * a NUL-terminated label ("histogram", "onesweep", "lds_row_sort", "transpose_last", ...) of
 * at most label_stride-1 characters at labels + i*label_stride, and the launch duration in
 * milliseconds at milliseconds[i], in launch order -- returns how many it wrote and forgets
 * all records (also those it had no room for).  Off by default; meant for benchmarks.  The
 * reference's counterpart is the Legate profiler range around each API call
 * (cupynumeric/_utils/profiling.py:37-73).
 */
int cpn_profile_enable(int on);
int cpn_profile_collect(char* labels, uint64_t label_stride, float* milliseconds, int max_records);

/*
 * Streaming-rate probe: one plain pass over `bytes` bytes (a multiple of 16, both pointers
 * 16-byte aligned) on `stream`, for benchmarks that want the device's own ceilings beside a
 * sort's rate.  mode CPN_STREAM_READ reads src (dst receives nothing unless the data holds one
 * improbable pattern, which keeps the loads alive), CPN_STREAM_COPY copies src to dst,
 * CPN_STREAM_FILL writes a constant to dst.  Loads and stores carry the nontemporal hint.
 * Returns 0 or a negative status.  No counterpart in the reference (its benchmarks time
 * whole API calls, examples/_benchmark/timer.py:199-241).
 */
#define CPN_STREAM_READ 0
#define CPN_STREAM_COPY 1
#define CPN_STREAM_FILL 2
int cpn_stream_probe(int mode, const void* src, void* dst, uint64_t bytes, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* CPN_SORT_H */
