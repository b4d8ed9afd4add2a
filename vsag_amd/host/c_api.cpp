// C entry points over the host index classes (the counterpart of the reference's src/vsag_c_api.cpp:194-333).
#include "vsag_host_c_api.h"

#include <algorithm>
#include <functional>
#include <cstdio>
#include <cstring>
#include <limits>
#include <memory>

#include "vsag_host.h"

namespace {

struct VsagIndex {
    explicit VsagIndex(std::shared_ptr<vsag::Index> index) : index_(std::move(index)) {
    }
    std::shared_ptr<vsag::Index> index_;
};

Error_t
make_error(int code, const std::string& message) {
    Error_t e;
    e.code = code;
    snprintf(e.message, sizeof(e.message), "%s", message.c_str());
    return e;
}

Error_t
make_error(const vsag::Error& error) {
    return make_error(-static_cast<int>(error.type), error.message);
}

const Error_t&
success() {
    static const Error_t ok = make_error(VSAG_SUCCESS, "success");
    return ok;
}

thread_local Error_t tl_factory_error = make_error(VSAG_SUCCESS, "success");
thread_local int64_t tl_failed_ids = 0;

vsag::DatasetPtr
base_dataset(const float* data, const int64_t* ids, uint64_t dim, uint64_t count) {
    auto dataset = vsag::Dataset::Make();
    dataset->Owner(false)
        ->Dim(static_cast<int64_t>(dim))
        ->NumElements(static_cast<int64_t>(count))
        ->Ids(ids)
        ->Float32Vectors(data);
    return dataset;
}

}  // namespace

extern "C" vsag_index_t
vsag_index_factory(const char* index_name, const char* index_param) {
    if (index_name == nullptr || index_param == nullptr) {
        tl_factory_error = make_error(VSAG_INVALID_ARGUMENT, "index name / parameters are NULL");
        return nullptr;
    }
    auto index = vsag::Factory::CreateIndex(index_name, index_param);
    if (index.has_value()) {
        tl_factory_error = success();
        return new VsagIndex(index.value());
    }
    tl_factory_error = make_error(index.error());
    return nullptr;
}

extern "C" Error_t
vsag_last_factory_error(void) {
    return tl_factory_error;
}

extern "C" Error_t
vsag_index_destroy(vsag_index_t index) {
    delete static_cast<VsagIndex*>(index);
    return success();
}

extern "C" Error_t
vsag_index_build(vsag_index_t index, const float* data, const int64_t* ids, uint64_t dim, uint64_t count) {
    auto* vi = static_cast<VsagIndex*>(index);
    if (vi == nullptr) {
        return make_error(VSAG_UNKNOWN_ERROR, "index is NULL");
    }
    auto result = vi->index_->Build(base_dataset(data, ids, dim, count));
    if (!result.has_value()) {
        return make_error(result.error());
    }
    tl_failed_ids = static_cast<int64_t>(result.value().size());
    return success();
}

extern "C" Error_t
vsag_index_add(vsag_index_t index, const float* data, const int64_t* ids, uint64_t dim, uint64_t count) {
    auto* vi = static_cast<VsagIndex*>(index);
    if (vi == nullptr) {
        return make_error(VSAG_UNKNOWN_ERROR, "index is NULL");
    }
    auto result = vi->index_->Add(base_dataset(data, ids, dim, count));
    if (!result.has_value()) {
        return make_error(result.error());
    }
    tl_failed_ids = static_cast<int64_t>(result.value().size());
    return success();
}

namespace {

// Shared body of the four single-query searches: `range` selects RangeSearch(radius, limited_size = k).
Error_t
search_one(vsag_index_t index, const float* query, uint64_t dim, bool range, float radius, int64_t k,
           const char* parameters, FilterFunc_t filter, SearchResult_t* search_result) {
    if (search_result == nullptr) {
        return make_error(VSAG_UNKNOWN_ERROR, "search result is NULL");
    }
    auto* vi = static_cast<VsagIndex*>(index);
    if (vi == nullptr) {
        return make_error(VSAG_UNKNOWN_ERROR, "index is NULL");
    }
    if (k <= 0) {
        return make_error(VSAG_INVALID_ARGUMENT, range ? "range_search requires k >= 1" : "knn_search requires k >= 1");
    }
    auto q = vsag::Dataset::Make();
    q->Owner(false)->Dim(static_cast<int64_t>(dim))->NumElements(1)->Float32Vectors(query);
    const std::string params = parameters ? parameters : "";
    std::function<bool(int64_t)> fn;
    if (filter != nullptr) {
        fn = [filter](int64_t id) { return filter(id); };
    }
    auto result = range ? (fn ? vi->index_->RangeSearch(q, radius, params, fn, k)
                              : vi->index_->RangeSearch(q, radius, params, k))
                        : (fn ? vi->index_->KnnSearch(q, k, params, fn) : vi->index_->KnnSearch(q, k, params));
    if (!result.has_value()) {
        return make_error(result.error());
    }
    int64_t to_write = std::min<int64_t>(result.value()->GetDim(), k);
    for (int64_t i = 0; i < to_write; ++i) {
        search_result->ids[i] = result.value()->GetIds()[i];
        search_result->dists[i] = result.value()->GetDistances()[i];
    }
    search_result->count = to_write;
    return success();
}

}  // namespace

extern "C" Error_t
vsag_index_knn_search(vsag_index_t index, const float* query, uint64_t dim, int64_t k, const char* parameters,
                      SearchResult_t* search_result) {
    return search_one(index, query, dim, false, 0.0F, k, parameters, nullptr, search_result);
}

extern "C" Error_t
vsag_index_knn_search_with_filter(vsag_index_t index, const float* query, uint64_t dim, int64_t k,
                                  const char* parameters, FilterFunc_t filter, SearchResult_t* search_result) {
    return search_one(index, query, dim, false, 0.0F, k, parameters, filter, search_result);
}

extern "C" Error_t
vsag_index_range_search(vsag_index_t index, const float* query, uint64_t dim, float radius, int64_t k,
                        const char* parameters, SearchResult_t* search_result) {
    return search_one(index, query, dim, true, radius, k, parameters, nullptr, search_result);
}

extern "C" Error_t
vsag_index_range_search_with_filter(vsag_index_t index, const float* query, uint64_t dim, float radius, int64_t k,
                                    const char* parameters, FilterFunc_t filter, SearchResult_t* search_result) {
    return search_one(index, query, dim, true, radius, k, parameters, filter, search_result);
}

extern "C" Error_t
vsag_index_knn_search_batch(vsag_index_t index, const float* queries, uint64_t nq, uint64_t dim, int64_t k,
                            const char* parameters, int64_t* ids, float* dists, int64_t* result_dim) {
    auto* vi = static_cast<VsagIndex*>(index);
    if (vi == nullptr) {
        return make_error(VSAG_UNKNOWN_ERROR, "index is NULL");
    }
    if (ids == nullptr || dists == nullptr) {
        return make_error(VSAG_INVALID_ARGUMENT, "result arrays are NULL");
    }
    auto q = vsag::Dataset::Make();
    q->Owner(false)->Dim(static_cast<int64_t>(dim))->NumElements(static_cast<int64_t>(nq))->Float32Vectors(queries);
    auto result = vi->index_->KnnSearch(q, k, parameters ? parameters : "");
    if (!result.has_value()) {
        return make_error(result.error());
    }
    const auto& r = result.value();
    const int64_t rows = r->GetNumElements(), cols = r->GetDim();
    for (uint64_t i = 0; i < nq; ++i) {
        for (int64_t j = 0; j < k; ++j) {
            bool have = static_cast<int64_t>(i) < rows && j < cols;
            ids[i * k + j] = have ? r->GetIds()[i * cols + j] : -1;
            dists[i * k + j] = have ? r->GetDistances()[i * cols + j] : std::numeric_limits<float>::infinity();
        }
    }
    if (result_dim != nullptr) {
        *result_dim = cols;
    }
    return success();
}

extern "C" int64_t
vsag_index_get_num_elements(vsag_index_t index) {
    auto* vi = static_cast<VsagIndex*>(index);
    return vi == nullptr ? 0 : vi->index_->GetNumElements();
}

extern "C" int64_t
vsag_last_failed_id_count(void) {
    return tl_failed_ids;
}
