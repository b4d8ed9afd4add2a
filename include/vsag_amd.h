/*
 * vsag_amd.h — C ABI of the MI355X (gfx950) search core that stands behind VSAG's brute_force / ivf
 * index classes.  Plain pointers and sizes only; every pointer named *_dev is device memory of the
 * current HIP device, everything else is host memory.  All functions return 0 or a negative VSAG_AMD_*
 * code (same values as VSAG_* in the reference's include/vsag/vsag_c_api.h:20-34) and leave a message
 * for vsag_amd_last_error() (thread-local).  Kernels are enqueued on `stream` (a hipStream_t passed as
 * void*, NULL = default stream) and the call returns without waiting unless stated otherwise.
 * Scratch memory is always supplied by the caller as (workspace_dev, workspace_bytes); the matching
 * *_workspace_bytes() function says how much a call needs.  Calls on different streams with different
 * workspaces may run concurrently on one store.
 *
 * Each entry point names the reference interface (file:line in the VSAG tree) it replaces.
 */
#ifndef VSAG_AMD_H
#define VSAG_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Exported entry points; everything else in the library has hidden visibility. */
#define VSAG_AMD_API __attribute__((visibility("default")))

#define VSAG_AMD_SUCCESS 0
#define VSAG_AMD_UNKNOWN_ERROR (-1)
#define VSAG_AMD_INTERNAL_ERROR (-2)
#define VSAG_AMD_INVALID_ARGUMENT (-3)
#define VSAG_AMD_WRONG_STATUS (-4)
#define VSAG_AMD_UNSUPPORTED_INDEX_OPERATION (-8)
#define VSAG_AMD_DIMENSION_NOT_EQUAL (-9)
#define VSAG_AMD_INDEX_EMPTY (-10)
#define VSAG_AMD_NO_ENOUGH_MEMORY (-11)

/* metric_type of the index JSON (src/constants.cpp:51-69): "l2" -> squared L2, "ip" -> 1 - <q,x>,
 * "cosine" -> 1 - cos. */
#define VSAG_AMD_METRIC_L2 0
#define VSAG_AMD_METRIC_IP 1
#define VSAG_AMD_METRIC_COSINE 2

/* base_quantization_type names of src/inner_string_params.h:90-102. */
#define VSAG_AMD_KIND_FP32 0
#define VSAG_AMD_KIND_SQ8 1
#define VSAG_AMD_KIND_SQ4 2
#define VSAG_AMD_KIND_SQ4_UNIFORM 3
#define VSAG_AMD_KIND_SQ8_UNIFORM 4
#define VSAG_AMD_KIND_RABITQ 5
#define VSAG_AMD_KIND_PQFS 6

/* SQTrainMode of src/quantization/scalar_quantization/scalar_quantization_trainer.h:24-28. */
#define VSAG_AMD_SQ_TRAIN_CLASSIC 1
#define VSAG_AMD_SQ_TRAIN_TRUNC_BOUND 3

#define VSAG_AMD_INVALID_ID 0xFFFFFFFFu

/* ------------------------------------------------------------------ runtime ------------------ */

/* Selects `device`, checks that it is a gfx950 part and that the library's code object loads.
 * Fails (VSAG_AMD_INTERNAL_ERROR) when there is no usable GPU: there is no CPU fallback. */
VSAG_AMD_API int vsag_amd_init(int device);
VSAG_AMD_API const char* vsag_amd_last_error(void);
/* Name of the device selected by vsag_amd_init, its CU count and memory (bytes). */
VSAG_AMD_API int vsag_amd_device_info(char* name, size_t name_bytes, int* compute_units, uint64_t* hbm_bytes);

/* Thin wrappers over hipMalloc / hipFree / hipMemcpyAsync / hipStreamSynchronize so that a host
 * with no HIP headers (cgo, ctypes, a C++ index class) can own device buffers.  The two copies that
 * touch host memory return after the copy has finished; d2d and memset are asynchronous. */
VSAG_AMD_API int vsag_amd_malloc(void** ptr_dev, size_t bytes);
VSAG_AMD_API int vsag_amd_free(void* ptr_dev);
/* Free and total device memory (hipMemGetInfo) and the high-water mark of the stream-ordered allocator's default
 * pool since it was last reset (reset_high != 0 resets it after reading): what a caller needs to check that a
 * call allocated nothing.  Any pointer may be NULL. */
VSAG_AMD_API int vsag_amd_memory_info(uint64_t* free_bytes, uint64_t* total_bytes, uint64_t* async_pool_high_bytes,
                                      int reset_high);
VSAG_AMD_API int vsag_amd_memcpy_h2d(void* dst_dev, const void* src, size_t bytes, void* stream);
VSAG_AMD_API int vsag_amd_memcpy_d2h(void* dst, const void* src_dev, size_t bytes, void* stream);
VSAG_AMD_API int vsag_amd_memcpy_d2d(void* dst_dev, const void* src_dev, size_t bytes, void* stream);
/* Pinned host memory (hipHostMalloc) and the two host copies without their wait: a search that stages its queries
 * and results through pinned buffers needs one vsag_amd_stream_synchronize, at its end.  With pageable host memory
 * the copies are still correct, but may block. */
VSAG_AMD_API int vsag_amd_host_malloc(void** ptr, size_t bytes);
VSAG_AMD_API int vsag_amd_host_free(void* ptr);
VSAG_AMD_API int vsag_amd_memcpy_h2d_async(void* dst_dev, const void* src, size_t bytes, void* stream);
VSAG_AMD_API int vsag_amd_memcpy_d2h_async(void* dst, const void* src_dev, size_t bytes, void* stream);
VSAG_AMD_API int vsag_amd_memset(void* dst_dev, int value, size_t bytes, void* stream);
VSAG_AMD_API int vsag_amd_stream_synchronize(void* stream);
/* A stream of default priority that does not synchronise with the null stream: one per concurrent search. */
VSAG_AMD_API int vsag_amd_stream_create(void** stream);
VSAG_AMD_API int vsag_amd_stream_destroy(void* stream);

/* ------------------------------------------------------------------ quantizer training ------- */

/* ScalarQuantizationTrainer::Train + ScalarQuantizer::TrainImpl
 * (scalar_quantization_trainer.cpp:30-45,89-146; scalar_quantizer.cpp:52-73): per-dimension lower bound
 * and diff = upper - lower from at most max_sample (0 = 100000) strided sample rows.  TRUNC_BOUND keeps
 * the ignore_count-th largest / smallest value per dimension; cosine normalises the sample rows first.
 * bits = 8 or 4.  Workspace: vsag_amd_sq_train_workspace_bytes(). */
VSAG_AMD_API size_t vsag_amd_sq_train_workspace_bytes(uint64_t n, uint32_t dim, uint64_t max_sample);
VSAG_AMD_API int vsag_amd_sq_train(const float* x_dev, uint64_t n, uint32_t dim, int bits, int metric, int mode,
                      float trunc_rate, uint64_t max_sample, float* lower_bound_dev, float* diff_dev,
                      void* workspace_dev, size_t workspace_bytes, void* stream);

/* ScalarQuantizationTrainer::TrainUniform + SQ4UniformQuantizer::TrainImpl / SQ8UniformQuantizer::
 * TrainImpl (scalar_quantization_trainer.cpp:47-70; sq4_uniform_quantizer.cpp:86-108;
 * sq8_uniform_quantizer.cpp:76-98).  Writes two floats: out_dev[0] = lower bound, out_dev[1] = diff. */
VSAG_AMD_API int vsag_amd_sq_train_uniform(const float* x_dev, uint64_t n, uint32_t dim, int bits, int metric,
                              int mode, float trunc_rate, uint64_t max_sample, float* out_dev,
                              void* workspace_dev, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ encoders ----------------- */

/* Bytes per code in the reference's layout (Quantizer::GetCodeSize): fp32 4*dim; sq8 dim; sq4
 * ceil(dim/2) (scalar_quantizer.cpp:28-36); uniform kinds sq4_uniform_quantizer.cpp:33-72 and
 * sq8_uniform_quantizer.cpp:30-62; rabitq rabitq_quantizer.cpp:102-133.  (pqfs: ceil(pq_dim / 2),
 * pq_fastscan_quantizer.cpp:38 -- it depends on pq_dim, not on dim: call it with dim = pq_dim.)
 *
 * Every `query_bits` / `rabitq_query_bits` argument of this header is a bits word: rabitq_bits_per_dim_query (4 or 32)
 * plus 256 * rabitq_bits_per_dim_base for multi-bit base codes (2..8 bits, fp32 queries only; 0 in the second byte
 * means 1 bit). */
#define VSAG_AMD_RABITQ_BITS(query_bits, base_bits) ((query_bits) | ((base_bits) > 1 ? (base_bits) << 8 : 0))
VSAG_AMD_API uint64_t vsag_amd_code_size(int kind, int metric, uint32_t dim, int rabitq_query_bits);

/* ScalarQuantizer::EncodeBatch (scalar_quantizer.cpp:85-112): fp32 rows -> sq8 / sq4 codes in the
 * reference byte layout, n x code_size.  Cosine normalises each row first. */
VSAG_AMD_API int vsag_amd_sq_encode(const float* x_dev, uint64_t n, uint32_t dim, int bits, int metric,
                       const float* lower_bound_dev, const float* diff_dev, uint8_t* codes_dev,
                       void* stream);

/* SQ4UniformQuantizer::EncodeOneImpl / SQ8UniformQuantizer::EncodeOneImpl
 * (sq4_uniform_quantizer.cpp:110-152, sq8_uniform_quantizer.cpp:100-132): codes plus the trailing
 * u64 sum of squared codes (L2) or f32 sums (IP / cosine).  bounds_dev = {lower bound, diff}.
 * Also used for queries (ProcessQueryImpl encodes the query with the same routine). */
VSAG_AMD_API int vsag_amd_squ_encode(const float* x_dev, uint64_t n, uint32_t dim, int bits, int metric,
                        const float* bounds_dev, uint8_t* codes_dev, void* stream);

/* RaBitQuantizer::TrainImpl (rabitq_quantizer.cpp:209-254) with the rotation supplied by the caller
 * (row-major dim x dim, y = R x): centroid = R * mean(x). */
VSAG_AMD_API int vsag_amd_rabitq_train(const float* x_dev, uint64_t n, uint32_t dim, const float* rotation_dev,
                          float* centroid_dev, void* stream);
/* RaBitQuantizer::EncodeOneInternal, 1-bit base (rabitq_quantizer.cpp:724-856): n x code_size codes
 * [bits | norm | error | sum (query_bits != 32) | raw norm (ip, cosine)]. */
VSAG_AMD_API int vsag_amd_rabitq_encode(const float* x_dev, uint64_t n, uint32_t dim, const float* rotation_dev,
                           const float* centroid_dev, int metric, int query_bits, uint8_t* codes_dev,
                           void* stream);
/* FhtKacRotator::Transform (src/impl/transform/fht_kac_rotate_transformer.cpp:64-96; `rabitq_use_fht`) as the dense
 * row-major rotation the rabitq entry points take: y = R x.  flip_host: 4 x ceil(dim / 8) bytes of sign bits (what
 * FhtKacRotator::Serialize writes); rotation_host: dim x dim floats.  Host memory on both sides, no device work. */
VSAG_AMD_API int vsag_amd_fht_kac_matrix(const uint8_t* flip_host, uint32_t dim, float* rotation_host);
/* RaBitQuantizer::DecodeOneImpl (rabitq_quantizer.cpp:871-899): n x dim floats, x = R^T ((+-1 / sqrt(dim)) norm + centroid).
 * 1-bit codes only (the reference returns false for the others: INVALID_ARGUMENT here).  bits_word as for the encoders. */
VSAG_AMD_API int vsag_amd_rabitq_decode(const uint8_t* codes_dev, uint64_t n, uint32_t dim, const float* rotation_dev,
                           const float* centroid_dev, int metric, int bits_word, float* out_dev, void* stream);
/* RaBitQuantizer::EncodeOneInternal, multi-bit base (rabitq_quantizer.cpp:774-809; bits_word =
 * VSAG_AMD_RABITQ_BITS(32, 2..8)): n x code_size codes [bit planes, plane b = bit b of every dimension (PackIntoPlanes,
 * :431-453) | norm of the centred code | norm | error | raw norm (ip, cosine)].  fast_encode chooses FastEncodeRaBitQ
 * (:609-704, the reference's default, fast_encode_rounds 1..32) over EncodeExtendRaBitQ (:455-607). */
VSAG_AMD_API int vsag_amd_rabitq_encode_multibit(const float* x_dev, uint64_t n, uint32_t dim, const float* rotation_dev,
                                    const float* centroid_dev, int metric, int bits_word, int fast_encode,
                                    uint32_t fast_encode_rounds, uint8_t* codes_dev, void* stream);
/* RaBitQuantizer::ProcessQueryImpl (rabitq_quantizer.cpp:2130-2217): nq x query_code_size processed
 * queries (4-bit: four bit planes of aligned_dim/8 bytes, lb, delta, code sum, norm, raw norm; fp32: the values, their
 * sum where the base code is multi-bit, norm, raw norm). */
VSAG_AMD_API uint64_t vsag_amd_rabitq_query_code_size(uint32_t dim, int metric, int query_bits);
VSAG_AMD_API int vsag_amd_rabitq_process_query(const float* q_dev, uint64_t nq, uint32_t dim,
                                  const float* rotation_dev, const float* centroid_dev, int metric,
                                  int query_bits, uint8_t* qcodes_dev, void* stream);

/* PQFastScanQuantizer (src/quantization/product_quantization/pq_fastscan_quantizer.cpp): pq_dim subspaces of
 * dim / pq_dim dimensions, 16 centroids each; codebooks_dev is pq_dim x 16 x (dim / pq_dim) floats.
 * vsag_amd_pq_train = TrainImpl (:62-94): 16 centroids per subspace from the first min(n, 65536) rows by k-means++ and
 * 25 Lloyd iterations (the reference's draws come from std::random_device; here subspace i draws from
 * mt19937(seed + i)); blocking.  vsag_amd_pq_encode = EncodeBatchImpl (:97-138): n x ceil(pq_dim / 2) code bytes,
 * subspace i in byte i / 2, low nibble for even i (norm_scratch_dev: n floats under cosine, else NULL).
 * vsag_amd_pq_decode = DecodeBatchImpl (:140-156).  vsag_amd_pqfs_process_query = ProcessQueryImpl (:299-361):
 * nq x (pq_dim * 16 + 8) bytes, the byte table of a query, then diff and lower bound as floats.
 * vsag_amd_pqfs_package / _unpack = Package32 / Unpack32 (:241-297) over ceil(n / 32) blocks of 32 codes, the order in
 * which BucketDataCell keeps and serializes pqfs codes (bucket_datacell.h:943-992). */
VSAG_AMD_API size_t vsag_amd_pq_train_workspace_bytes(uint64_t n, uint32_t dim, uint32_t pq_dim);
VSAG_AMD_API int vsag_amd_pq_train(const float* x_dev, uint64_t n, uint32_t dim, uint32_t pq_dim, int metric, uint64_t seed,
                      float* codebooks_dev, void* workspace_dev, size_t workspace_bytes, void* stream);
VSAG_AMD_API int vsag_amd_pq_encode(const float* x_dev, uint64_t n, uint32_t dim, uint32_t pq_dim, const float* codebooks_dev,
                       int metric, uint8_t* codes_dev, float* norm_scratch_dev, void* stream);
VSAG_AMD_API int vsag_amd_pq_decode(const uint8_t* codes_dev, uint64_t n, uint32_t dim, uint32_t pq_dim,
                       const float* codebooks_dev, float* out_dev, void* stream);
VSAG_AMD_API int vsag_amd_pqfs_process_query(const float* q_dev, uint64_t nq, uint32_t dim, uint32_t pq_dim,
                                const float* codebooks_dev, int metric, uint8_t* qcodes_dev, void* stream);
VSAG_AMD_API int vsag_amd_pqfs_package(const uint8_t* codes_dev, uint64_t n, uint32_t pq_dim, uint8_t* packaged_dev,
                          void* stream);
VSAG_AMD_API int vsag_amd_pqfs_unpack(const uint8_t* packaged_dev, uint64_t n, uint32_t pq_dim, uint8_t* codes_dev,
                         void* stream);

/* ------------------------------------------------------------------ code stores -------------- */

/* A store is the device-resident replacement of one FlattenDataCell / BucketDataCell
 * (src/datacell/flatten_datacell.h:262-314, src/datacell/bucket_datacell.h:670-709): it keeps the
 * quantizer state and the codes re-tiled for coalesced wave64 reads (64 codes per tile, 16-byte
 * granules interleaved across lanes). */
typedef struct vsag_amd_store vsag_amd_store_t;

typedef struct vsag_amd_store_params {
    int kind;                    /* VSAG_AMD_KIND_* */
    int metric;                  /* VSAG_AMD_METRIC_* */
    uint32_t dim;
    const float* lower_bound_dev; /* sq8/sq4: dim floats.  uniform kinds: bounds {lb, diff}. */
    const float* diff_dev;        /* sq8/sq4: dim floats.  otherwise NULL. */
    const float* rotation_dev;    /* rabitq: dim x dim row-major.  otherwise NULL. */
    const float* centroid_dev;    /* rabitq: dim floats (already rotated). */
    int rabitq_query_bits;        /* rabitq: the bits word, VSAG_AMD_RABITQ_BITS(4 | 32, base bits); 0 = 4-bit queries. */
    uint32_t pq_dim;              /* pqfs: number of subspaces (divides dim, at most 1024). */
    const float* codebooks_dev;   /* pqfs: pq_dim x 16 x (dim / pq_dim) floats. */
} vsag_amd_store_params_t;

VSAG_AMD_API int vsag_amd_store_create(const vsag_amd_store_params_t* params, vsag_amd_store_t** store);
VSAG_AMD_API int vsag_amd_store_destroy(vsag_amd_store_t* store);
VSAG_AMD_API uint64_t vsag_amd_store_size(const vsag_amd_store_t* store);

/* FlattenDataCell::BatchInsertVector (flatten_datacell.h:279-314): append n codes given in the
 * reference byte layout (n x code_size, device memory); inner ids continue from the current size.
 * Synchronises `stream` when the store has to grow. */
VSAG_AMD_API int vsag_amd_store_append(vsag_amd_store_t* store, const uint8_t* codes_dev, uint64_t n, void* stream);

/* Posting-list form (BucketDataCell, bucket_datacell.h:670-709 + IVF::Add, ivf.cpp:590-724): codes in
 * the reference byte layout in inner-id order plus one bucket label per code.  Lists are laid out
 * contiguously, each padded to whole tiles, in stable (input) order inside a bucket.  Replaces any
 * previous content. */
VSAG_AMD_API int vsag_amd_store_set_lists(vsag_amd_store_t* store, const uint8_t* codes_dev, const int32_t* labels_dev,
                             uint64_t n, uint32_t nlist, void* stream);
/* IVF::Add on a filled index (ivf.cpp:590-724, BucketDataCell::InsertVector, bucket_datacell.h:670-709): n more codes
 * (reference byte layout; source row r gets inner id size + r) go behind the codes their lists already hold, in input
 * order.  Lists have some room behind their last tile; when one outgrows it, all lists move once to a layout with a
 * quarter more room.  residual_bias_dev: per source row, for stores with residual centroids and the l2 metric
 * (vsag_amd_residual_bias), else NULL.  Blocking. */
VSAG_AMD_API int vsag_amd_store_append_lists(vsag_amd_store_t* store, const uint8_t* codes_dev, const int32_t* labels_dev,
                                const float* residual_bias_dev, uint64_t n, void* stream);

/* use_residual of BucketDataCell (bucket_datacell.h:527-572,594-639): the lists hold codes of x - c, c the centroid of
 * the list (x normalised first for cosine), and a scan puts every distance right with the slot's bias and <q, c>.
 * vsag_amd_store_set_residual copies the nlist x dim centroids into an empty store (before vsag_amd_store_set_lists with
 * n = 0 and vsag_amd_store_append_lists); vsag_amd_residual_rows writes x_i - c[labels_i]; vsag_amd_residual_bias
 * decodes the codes (DecodeOneImpl of fp32 / sq8 / sq4 / sq8_uniform / sq4_uniform) into decoded_dev (n x dim floats of
 * scratch) and writes -2 <c, decoded> - <c, c> per row (encode_vector, bucket_datacell.h:626-636; l2 only). */
VSAG_AMD_API int vsag_amd_store_set_residual(vsag_amd_store_t* store, const float* centroids_dev, uint32_t nlist, void* stream);
VSAG_AMD_API int vsag_amd_residual_rows(const float* x_dev, uint64_t n, uint32_t dim, int metric, const int32_t* labels_dev,
                           const float* centroids_dev, float* out_dev, void* stream);
VSAG_AMD_API int vsag_amd_residual_bias(const vsag_amd_store_t* store, const uint8_t* codes_dev, uint64_t n,
                           const int32_t* labels_dev, const float* centroids_dev, float* bias_dev, float* decoded_dev,
                           void* stream);

/* The payload of FlattenDataCell::Serialize (flatten_datacell.h:481-486, io/common/basic_io.h:196-207): codes
 * [first, first + n) of a flat store back in the reference byte layout (n x code_size bytes).  The store keeps the
 * u64 sums of squares of the uniform kinds as floats; the exported code carries them recomputed from its bytes. */
VSAG_AMD_API int vsag_amd_store_export_codes(const vsag_amd_store_t* store, uint64_t first, uint64_t n, uint8_t* codes_dev,
                                void* stream);
/* The payload of BucketDataCell::Serialize (bucket_datacell.h:892-904): every list's codes, list by list in list
 * order (vsag_amd_store_list_sizes gives the cuts), with their inner ids and, for residual stores with the l2 metric,
 * their bias (bias_dev may be NULL).  Blocking. */
VSAG_AMD_API int vsag_amd_store_export_lists(const vsag_amd_store_t* store, uint8_t* codes_dev, uint32_t* ids_dev,
                                float* bias_dev, void* stream);

/* Deserialize (flatten_datacell.h:488-497): while on, appended codes are taken as they were exported -- an fp32 store
 * under cosine does not normalise rows that are unit vectors already. */
VSAG_AMD_API int vsag_amd_store_expect_stored_codes(vsag_amd_store_t* store, int on);

/* Sizes of the posting lists (nlist values) copied to host memory. */
VSAG_AMD_API int vsag_amd_store_list_sizes(const vsag_amd_store_t* store, uint32_t* sizes, uint32_t nlist);

/* FlattenDataCell::Query / BucketDataCell::QueryOneById (flatten_datacell.h:334-440, bucket_datacell.h:353-383; what
 * Index::CalDistanceById and a reorder over quantised codes call): distance of query i to each of its own `count`
 * codes named by inner id (ids_dev: nq x count; VSAG_AMD_INVALID_ID or an id the store does not hold gives -1).
 * Same arithmetic as the scans.  nq <= 65535. */
VSAG_AMD_API size_t vsag_amd_store_distances_workspace_bytes(const vsag_amd_store_t* store, uint64_t nq);
VSAG_AMD_API int vsag_amd_store_distances(const vsag_amd_store_t* store, const float* queries_dev, uint64_t nq,
                             const uint32_t* ids_dev, uint32_t count, float* dists_dev, void* workspace_dev,
                             size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ flat scan + top-k -------- */

/* BruteForce::SearchWithRequest hot loop (bruteforce.cpp:481-597) = FlattenDataCell::query
 * (flatten_datacell.h:334-440) + Quantizer::ComputeDistImpl + DistanceHeap (impl/heap/), batched over
 * queries.  queries_dev: nq x dim fp32 raw queries (the library applies ProcessQueryImpl of the store's
 * quantizer itself).  Output: nq x k inner ids / distances, ascending by (distance, id); rows shorter
 * than k are padded with VSAG_AMD_INVALID_ID / +inf.  1 <= k <= 1024. */
VSAG_AMD_API size_t vsag_amd_flat_scan_workspace_bytes(const vsag_amd_store_t* store, uint64_t nq, uint32_t k);
VSAG_AMD_API int vsag_amd_flat_scan_topk(const vsag_amd_store_t* store, const float* queries_dev, uint64_t nq,
                            uint32_t k, uint32_t* ids_dev, float* dists_dev, void* workspace_dev,
                            size_t workspace_bytes, void* stream);

/* Pre-filter and range limit of a search (BruteForce::SearchWithRequest with a Filter and in RANGE_SEARCH mode,
 * bruteforce.cpp:519-545; FlatBucketSearcher::Search, flat_bucket_searcher.cpp:61-137).
 * deny_bits_dev: bit (id & 31) of word (id >> 5) set = inner id `id` is filtered out, ceil(n / 32) words of
 * device memory, or NULL.  The caller maps labels to inner ids (InnerIdWrapperFilter,
 * impl/filter/inner_id_wrapper_filter.h:23-57).  use_radius != 0: only distances <= radius are returned. */
typedef struct vsag_amd_search_options {
    const uint32_t* deny_bits_dev;
    int use_radius;
    float radius;
} vsag_amd_search_options_t;

/* vsag_amd_flat_scan_topk under the given options (NULL = none).  Same workspace size. */
VSAG_AMD_API int vsag_amd_flat_scan_topk_ex(const vsag_amd_store_t* store, const float* queries_dev, uint64_t nq,
                               uint32_t k, const vsag_amd_search_options_t* options, uint32_t* ids_dev,
                               float* dists_dev, void* workspace_dev, size_t workspace_bytes, void* stream);

/* vsag_amd_flat_scan_topk_ex without a workspace argument and without any allocation: the scan's intermediate
 * buffers live in a scratch array inside the library's device image (vsag_amd_flat_scan_noalloc_max_bytes() bytes,
 * 32 MiB, held on every GPU the library runs on until the process ends).  No counterpart in the reference; it is for
 * callers that cannot call hipMalloc -- code under HIP graph capture, tight serving loops, harnesses that forbid
 * allocation.  Same results as vsag_amd_flat_scan_topk_ex (options may be NULL).  A scan whose
 * vsag_amd_flat_scan_workspace_bytes() exceeds the array is rejected with VSAG_AMD_INVALID_ARGUMENT (10^6 sq8 codes
 * and k = 10: about a thousand queries per call fit).  All calls on one GPU share the array: calls that overlap on
 * one GPU race, whatever their streams.  Calls no hipMalloc / hipFree and creates no events (the measurement hook is
 * off for the call). */
VSAG_AMD_API size_t vsag_amd_flat_scan_noalloc_max_bytes(void);
VSAG_AMD_API int vsag_amd_flat_scan_topk_noalloc(const vsag_amd_store_t* store, const float* queries_dev, uint64_t nq,
                                    uint32_t k, const vsag_amd_search_options_t* options, uint32_t* ids_dev,
                                    float* dists_dev, void* stream);

/* Large batches on flat fp32 / sq8 / sq8_uniform / sq4_uniform (the uniform kinds: at most 128 dimensions) / rabitq stores are served by a matrix-core contraction that pre-selects
 * candidates, which are then recomputed and selected exactly as the streaming scan does (same results, bit for bit).
 * rabitq stores with 4-bit queries and at most 1024 dimensions (L2, inner product) expand code bits and query nibbles to
 * bytes for the int8 matrix cores (the integer product is exact; k up to 256 by default).
 * Posting lists of sq4_uniform codes of at most 128 dimensions (any metric) scan the probe columns behind the first on the
 * int8 matrix cores when a batch has at least 8192 (query, list) groups (same results; off with mode -1).
 * sq8 stores of at most 128 dimensions pre-select on the int8 matrix cores (queries split into two int8 planes
 * with a rigorous bound on the remainder), the others on the fp32 matrix cores.
 * mode: 0 = when it pays (default: >= 512 queries, k <= 128, >= 65536 codes), 1 = whenever the store and k
 * allow it, 2 = like 1 but always on the fp32 matrix cores, -1 = never.  Process-wide; affects
 * vsag_amd_flat_scan_workspace_bytes as well.  No counterpart in the reference (it scans one query at a time). */
VSAG_AMD_API int vsag_amd_set_scan_contraction(int mode);

/* Tuning knobs of the scan (query tile T in {1,2,4,8}, 0 = automatic; number of base chunks, 0 =
 * automatic).  Process-wide; meant for benchmarks. */
VSAG_AMD_API int vsag_amd_set_scan_tuning(int query_tile, int base_chunks);

/* The same two settings for one store; they go before the process-wide ones, so that callers with different needs can
 * share a process (and searches on other stores are not disturbed by a change).  mode -2 / query_tile -1 /
 * base_chunks -1 = follow the process-wide setting (the default).  Set them while no search runs on the store.  No
 * counterpart in the reference. */
VSAG_AMD_API int vsag_amd_store_set_scan_contraction(vsag_amd_store_t* store, int mode);
VSAG_AMD_API int vsag_amd_store_set_scan_tuning(vsag_amd_store_t* store, int query_tile, int base_chunks);
/* What the last flat scan on this thread used: query tile (128 / 256: the batch went through the fp32 / int8
 * matrix cores), passes over the code array, bytes of codes one pass reads.  After a posting-list scan: query tile
 * only (256: the columns behind the first went through the int8 matrix cores). */
VSAG_AMD_API int vsag_amd_last_scan_info(int* query_tile, uint64_t* passes, uint64_t* bytes_per_pass);

/* Measurement hook: when enabled, a call records HIP events on its stream around the launch of its
 * dominant kernel (flat scan, posting-list scan, k-means assignment); vsag_amd_last_kernel_ms() waits
 * for the last such launch of the calling thread and returns its duration. */
VSAG_AMD_API int vsag_amd_set_kernel_timing(int enable);
VSAG_AMD_API int vsag_amd_last_kernel_ms(float* ms);

/* ------------------------------------------------------------------ k-means ------------------ */

/* KMeansCluster::find_nearest_one_with_blas (impl/cluster/kmeans_cluster.cpp:193-305):
 * labels[i] = first argmin_j (||c_j||^2 - 2<c_j, x_i>), min_dist[i] = that minimum (may be NULL),
 * *loss_dev (double, may be NULL) = sum_i (min + ||x_i||^2) / n. */
VSAG_AMD_API size_t vsag_amd_kmeans_assign_workspace_bytes(uint64_t n, uint32_t dim, uint32_t k);
VSAG_AMD_API int vsag_amd_kmeans_assign(const float* x_dev, uint64_t n, uint32_t dim, const float* centroids_dev,
                           uint32_t k, int32_t* labels_dev, float* min_dist_dev, double* loss_dev,
                           void* workspace_dev, size_t workspace_bytes, void* stream);
/* Centroid update of KMeansCluster::Run (kmeans_cluster.cpp:108-172): mean of member rows; clusters
 * with no member keep their centroid and report counts_dev[j] = 0 (the caller re-seeds them). */
VSAG_AMD_API size_t vsag_amd_kmeans_update_workspace_bytes(uint64_t n, uint32_t dim, uint32_t k);
VSAG_AMD_API int vsag_amd_kmeans_update(const float* x_dev, const int32_t* labels_dev, uint64_t n, uint32_t dim,
                           uint32_t k, float* centroids_dev, int32_t* counts_dev, void* workspace_dev,
                           size_t workspace_bytes, void* stream);
/* KMeansCluster::Run (kmeans_cluster.cpp:46-190) with the initial centroids given in centroids_dev
 * and empty clusters re-seeded from mt19937(seed) (the reference draws both from std::random_device).
 * Runs `iters` Lloyd iterations; *loss receives the loss of the last assignment.  Blocking. */
VSAG_AMD_API size_t vsag_amd_kmeans_run_workspace_bytes(uint64_t n, uint32_t dim, uint32_t k);
VSAG_AMD_API int vsag_amd_kmeans_run(const float* x_dev, uint64_t n, uint32_t dim, float* centroids_dev, uint32_t k,
                        int iters, uint64_t seed, int32_t* labels_dev, double* loss,
                        void* workspace_dev, size_t workspace_bytes, void* stream);

/* KMeansCluster::select_initial_centroids_kmeans_plus_plus (kmeans_cluster.cpp:383-435), the reference's default
 * initialisation, with its random draws as inputs (the reference takes them from an mt19937 seeded by
 * std::random_device): `first` = the row that becomes centroid 0; draws (HOST array, k - 1 doubles in [0, 1)): centroid
 * j is the first row at which the running sum of the rows' smallest squared distances to the centroids so far reaches
 * draws[j - 1] * their total (any row, floor(draw * n), when the total is 0).  picks_dev (k words, may be NULL) receives
 * the chosen rows. */
VSAG_AMD_API size_t vsag_amd_kmeans_init_plus_plus_workspace_bytes(uint64_t n);
VSAG_AMD_API int vsag_amd_kmeans_init_plus_plus(const float* x_dev, uint64_t n, uint32_t dim, uint32_t k, uint64_t first,
                                   const double* draws, float* centroids_dev, uint64_t* picks_dev,
                                   void* workspace_dev, size_t workspace_bytes, void* stream);

/* ------------------------------------------------------------------ IVF ---------------------- */

/* Routing (IVFNearestPartition::ClassifyDatasForSearch, ivf_nearest_partition.cpp:99-147, done exactly
 * instead of through the reference's HGraph): the nprobe nearest centroids of every query, ascending.
 * centroids are an fp32 store created with vsag_amd_store_create + append.  From 1024 queries on, 1024 to 8192
 * centroids are ranked through a table of approximate distances (nq x centroids x 4 bytes of the workspace) and the
 * ones that can be among the nprobe nearest are scored exactly: the same buckets and distances as for fewer queries. */
VSAG_AMD_API size_t vsag_amd_ivf_route_workspace_bytes(const vsag_amd_store_t* centroids, uint64_t nq, uint32_t nprobe);
VSAG_AMD_API int vsag_amd_ivf_route(const vsag_amd_store_t* centroids, const float* queries_dev, uint64_t nq,
                       uint32_t nprobe, int32_t* buckets_dev, float* dists_dev, void* workspace_dev,
                       size_t workspace_bytes, void* stream);

/* IVF::search<KNN_SEARCH> (ivf.cpp:1693-1828) = BucketDataCell::ScanBucketById
 * (bucket_datacell.h:527-572) + FlatBucketSearcher::Search (flat_bucket_searcher.cpp:26-138) for a
 * batch: every query scans the nprobe lists named in buckets_dev (nq x nprobe, -1 = skip) and keeps the
 * kcand best (distance, inner id), ascending, padded with VSAG_AMD_INVALID_ID / +inf. */
VSAG_AMD_API size_t vsag_amd_ivf_scan_workspace_bytes(const vsag_amd_store_t* lists, uint64_t nq, uint32_t nprobe,
                                         uint32_t kcand);
VSAG_AMD_API int vsag_amd_ivf_scan_topk(const vsag_amd_store_t* lists, const float* queries_dev, uint64_t nq,
                           const int32_t* buckets_dev, uint32_t nprobe, uint32_t kcand, uint32_t* ids_dev,
                           float* dists_dev, void* workspace_dev, size_t workspace_bytes, void* stream);

/* vsag_amd_ivf_scan_topk under the given options (NULL = none).  Same workspace size. */
VSAG_AMD_API int vsag_amd_ivf_scan_topk_ex(const vsag_amd_store_t* lists, const float* queries_dev, uint64_t nq,
                              const int32_t* buckets_dev, uint32_t nprobe, uint32_t kcand,
                              const vsag_amd_search_options_t* options, uint32_t* ids_dev, float* dists_dev,
                              void* workspace_dev, size_t workspace_bytes, void* stream);

/* Number of codes in the lists a batch probes, summed over all (query, probe) pairs: the approximate-phase
 * distance_evaluations of SearchStatistics (src/query_context.h:215-246).  total_dev: 8 bytes of device memory. */
VSAG_AMD_API int vsag_amd_ivf_probed_codes(const vsag_amd_store_t* lists, const int32_t* buckets_dev, uint64_t nq,
                              uint32_t nprobe, uint64_t* total_dev, void* stream);

/* FlattenReorder::Reorder (impl/reorder/flatten_reorder.cpp:52-114): exact fp32 distances of the
 * candidates (nq x kcand inner ids into raw_dev, n x dim fp32 row-major; VSAG_AMD_INVALID_ID skipped),
 * best k kept, ascending. */
VSAG_AMD_API int vsag_amd_rerank_fp32(const float* raw_dev, uint64_t n, uint32_t dim, int metric,
                         const float* queries_dev, uint64_t nq, const uint32_t* cand_ids_dev,
                         uint32_t kcand, uint32_t k, uint32_t* ids_dev, float* dists_dev, void* stream);

/* FlattenDataCell::Query over fp32 codes (flatten_datacell.h:334-440; IVF::CalDistanceById with precise distances,
 * ivf.cpp:2462-2465): the exact distance of every (query, inner id) pair in the order given, nq x count, with the
 * arithmetic of vsag_amd_rerank_fp32; -1 where the id is VSAG_AMD_INVALID_ID or beyond the rows. */
VSAG_AMD_API int vsag_amd_rows_distances_fp32(const float* raw_dev, uint64_t n, uint32_t dim, int metric,
                                 const float* queries_dev, uint64_t nq, const uint32_t* ids_dev, uint32_t count,
                                 float* dists_dev, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* VSAG_AMD_H */
