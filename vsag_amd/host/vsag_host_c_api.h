/* C view of the host layer, shaped like the reference's include/vsag/vsag_c_api.h:20-160 (same error
 * codes, Error_t by value, caller-owned result arrays), so that a program written against the reference's
 * C API drives the GPU-backed index classes unchanged.  vsag_index_knn_search_batch is the only addition:
 * the reference's C entry point takes one query per call. */
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
VSAG_HOST_API int64_t vsag_index_get_num_elements(vsag_index_t index);
/* Number of ids the last build / add on this thread could not insert (duplicates). */
VSAG_HOST_API int64_t vsag_last_failed_id_count(void);

#ifdef __cplusplus
}
#endif

#endif /* VSAG_HOST_C_API_H */
