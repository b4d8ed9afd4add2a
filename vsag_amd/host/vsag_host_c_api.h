/* C view of the host layer, shaped like the reference's include/vsag/vsag_c_api.h:20-160 (same error
 * codes, Error_t by value, caller-owned result arrays), so that a program written against the reference's
 * C API drives the GPU-backed index classes unchanged.  Additions, marked below: vsag_index_knn_search_batch and
 * vsag_index_search_buckets (the reference's C entry points take one query per call and cannot name buckets), and
 * vsag_index_calculate_distances (rows of queries, precise / top-k selection of Index::CalDistanceById). */
#ifndef VSAG_HOST_C_API_H
#define VSAG_HOST_C_API_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VSAG_SUCCESS 0
#define VSAG_UNKNOWN_ERROR -1
#define VSAG_INTERNAL_ERROR -2
#define VSAG_INVALID_ARGUMENT -3
#define VSAG_WRONG_STATUS -4
#define VSAG_BUILD_TWICE -5
#define VSAG_INDEX_NOT_EMPTY -6
#define VSAG_UNSUPPORTED_INDEX -7
#define VSAG_UNSUPPORTED_INDEX_OPERATION -8
#define VSAG_DIMENSION_NOT_EQUAL -9
#define VSAG_INDEX_EMPTY -10
#define VSAG_NO_ENOUGH_MEMORY -11
#define VSAG_READ_ERROR -12
#define VSAG_MISSING_FILE -13
#define VSAG_INVALID_BINARY -14

typedef struct Error {
    int code;
    char message[1024];
} Error_t;

typedef void* vsag_index_t;

typedef struct SearchResult {
    float* dists;       /* caller-owned, room for k values */
    int64_t* ids;       /* caller-owned, room for k values */
    int64_t count;      /* results written */
    void* other_result; /* unused here */
} SearchResult_t;

#define VSAG_HOST_API __attribute__((visibility("default")))

/* Returns NULL on failure; vsag_last_factory_error() then holds the reason (the reference drops it). */
VSAG_HOST_API vsag_index_t vsag_index_factory(const char* index_name, const char* index_param);
VSAG_HOST_API Error_t vsag_last_factory_error(void);
VSAG_HOST_API Error_t vsag_index_destroy(vsag_index_t index);
VSAG_HOST_API Error_t vsag_index_build(vsag_index_t index, const float* data, const int64_t* ids, uint64_t dim,
                                       uint64_t count);
VSAG_HOST_API Error_t vsag_index_add(vsag_index_t index, const float* data, const int64_t* ids, uint64_t dim,
                                     uint64_t count);
VSAG_HOST_API Error_t vsag_index_knn_search(vsag_index_t index, const float* query, uint64_t dim, int64_t k,
                                            const char* parameters, SearchResult_t* search_result);
/* filter(label) == true filters the vector out (include/vsag/vsag_c_api.h:43,165-172). */
typedef bool (*FilterFunc_t)(int64_t id);
VSAG_HOST_API Error_t vsag_index_knn_search_with_filter(vsag_index_t index, const float* query, uint64_t dim, int64_t k,
                                                        const char* parameters, FilterFunc_t filter,
                                                        SearchResult_t* search_result);
/* Everything within radius, at most k (>= 1) results, nearest first (vsag_c_api.h:186-216). */
VSAG_HOST_API Error_t vsag_index_range_search(vsag_index_t index, const float* query, uint64_t dim, float radius,
                                              int64_t k, const char* parameters, SearchResult_t* search_result);
VSAG_HOST_API Error_t vsag_index_range_search_with_filter(vsag_index_t index, const float* query, uint64_t dim,
                                                          float radius, int64_t k, const char* parameters,
                                                          FilterFunc_t filter, SearchResult_t* search_result);
/* nq queries at once; ids / dists have room for nq * k values, rows padded with -1 / +inf. */
VSAG_HOST_API Error_t vsag_index_knn_search_batch(vsag_index_t index, const float* queries, uint64_t nq, uint64_t dim,
                                                  int64_t k, const char* parameters, int64_t* ids, float* dists,
                                                  int64_t* result_dim);
/* Addition: Index::SearchWithRequest with bucket_ids_ (include/vsag/search_request.h): query i scans the lists
 * bucket_ids[bucket_offsets[i] .. bucket_offsets[i + 1]) instead of the routed ones; bucket_offsets has nq + 1 entries
 * (NULL: default routing).  Output as vsag_index_knn_search_batch. */
VSAG_HOST_API Error_t vsag_index_search_buckets(vsag_index_t index, const float* queries, uint64_t nq, uint64_t dim,
                                                int64_t k, const char* parameters, const int64_t* bucket_ids,
                                                const uint64_t* bucket_offsets, int64_t* ids, float* dists,
                                                int64_t* result_dim);
/* include/vsag/vsag_c_api.h:128-133: trains the index (centroids, quantizers); no data is added. */
VSAG_HOST_API Error_t vsag_index_train(vsag_index_t index, const float* data, const int64_t* ids, uint64_t dim,
                                       uint64_t count);
/* include/vsag/vsag_c_api.h:250-255: distances between the query and the vectors with the given labels, in the order
 * of `ids`; -1 for a label the index does not hold. */
VSAG_HOST_API Error_t vsag_index_calculate_distance_by_ids(vsag_index_t index, const float* query, uint64_t dim,
                                                           const int64_t* ids, uint64_t count, float* dists);
/* Addition: Index::CalDistanceById in full (include/vsag/index.h:575-633): nq queries, row i against
 * ids[i * count ...]; topk == -1 writes nq x count distances in the order of ids (out_ids may be NULL), topk > 0 the
 * min(topk, count) smallest per row with their labels. */
VSAG_HOST_API Error_t vsag_index_calculate_distances(vsag_index_t index, const float* queries, uint64_t nq, uint64_t dim,
                                                     const int64_t* ids, uint64_t count, bool precise, int64_t topk,
                                                     int64_t* out_ids, float* out_dists);
/* include/vsag/vsag_c_api.h:50-65: statistics of the next search that writes search_result (a JSON string with
 * dist_cmp, distance_evaluations_by_phase, ...; NULL when none were recorded). */
VSAG_HOST_API Error_t vsag_search_result_enable_statistics(SearchResult_t* search_result);
VSAG_HOST_API const char* vsag_search_result_get_statistics(const SearchResult_t* search_result);
VSAG_HOST_API void vsag_search_result_destroy_statistics(SearchResult_t* search_result);
/* include/vsag/vsag_c_api.h:327-330: the index to a file (Index::Serialize(std::ostream&)) and back into an empty
 * index made with the same parameters. */
VSAG_HOST_API Error_t vsag_serialize_file(vsag_index_t index, const char* file_path);
VSAG_HOST_API Error_t vsag_deserialize_file(vsag_index_t index, const char* file_path);
/* Addition: the search loop of the reference's evaluator (tools/eval/case/search_eval_case.cpp:233-277): one query
 * per KnnSearch call, the queries handed out dynamically to `threads` caller threads that share the index; ids and
 * distances as vsag_index_knn_search_batch writes them, the wall-clock seconds of the loop in *seconds. */
VSAG_HOST_API Error_t vsag_index_eval_knn_search(vsag_index_t index, const float* queries, uint64_t nq, uint64_t dim,
                                                 int64_t k, const char* parameters, int threads, int64_t* ids,
                                                 float* dists, double* seconds);
VSAG_HOST_API int64_t vsag_index_get_num_elements(vsag_index_t index);
/* Number of ids the last build / add on this thread could not insert (duplicates). */
VSAG_HOST_API int64_t vsag_last_failed_id_count(void);

#ifdef __cplusplus
}
#endif

#endif /* VSAG_HOST_C_API_H */
