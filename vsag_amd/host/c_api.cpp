// C entry points over the host index classes (the counterpart of the reference's src/vsag_c_api.cpp:194-333).
#include "vsag_host_c_api.h"

#include <algorithm>
#include <atomic>
#include <chrono>
#include <thread>
#include <vector>
#include <functional>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <limits>
#include <memory>
#include <mutex>
#include <unordered_map>
#include <unordered_set>

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

// src/vsag_c_api.cpp:70-140: statistics are kept per SearchResult_t that asked for them.
std::mutex statistics_mutex;
std::unordered_set<const SearchResult_t*> statistics_requests;
std::unordered_map<const SearchResult_t*, std::unique_ptr<std::string>> statistics_results;

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
    {
        std::lock_guard<std::mutex> lock(statistics_mutex);
        if (statistics_requests.erase(search_result) != 0) {
            statistics_results[search_result] = std::make_unique<std::string>(result.value()->GetStatistics());
        }
    }
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

extern "C" Error_t
vsag_index_eval_knn_search(vsag_index_t index, const float* queries, uint64_t nq, uint64_t dim, int64_t k,
                           const char* parameters, int threads, int64_t* ids, float* dists, double* seconds) {
    auto* vi = static_cast<VsagIndex*>(index);
    if (vi == nullptr) {
        return make_error(VSAG_UNKNOWN_ERROR, "index is NULL");
    }
    if (ids == nullptr || dists == nullptr || queries == nullptr || k <= 0 || threads <= 0) {
        return make_error(VSAG_INVALID_ARGUMENT, "null array, k or thread count not positive");
    }
    const std::string params = parameters ? parameters : "";
    std::atomic<uint64_t> next{0};
    std::mutex error_mutex;
    bool failed = false;
    vsag::Error first_error(vsag::ErrorType::UNKNOWN_ERROR, "");
    auto worker = [&]() {
        for (;;) {
            const uint64_t i = next.fetch_add(1);
            if (i >= nq) {
                return;
            }
            auto q = vsag::Dataset::Make();
            q->Owner(false)->Dim(static_cast<int64_t>(dim))->NumElements(1)->Float32Vectors(queries + i * dim);
            auto result = vi->index_->KnnSearch(q, k, params);
            if (!result.has_value()) {
                std::lock_guard<std::mutex> lock(error_mutex);
                if (!failed) {
                    failed = true;
                    first_error = result.error();
                }
                return;
            }
            const auto& r = result.value();
            const int64_t cols = r->GetDim();
            for (int64_t j = 0; j < k; ++j) {
                const bool have = r->GetNumElements() > 0 && j < cols;
                ids[i * k + j] = have ? r->GetIds()[j] : -1;
                dists[i * k + j] = have ? r->GetDistances()[j] : std::numeric_limits<float>::infinity();
            }
        }
    };
    const auto t0 = std::chrono::steady_clock::now();
    std::vector<std::thread> pool;
    for (int t = 1; t < threads; ++t) {
        pool.emplace_back(worker);
    }
    worker();
    for (auto& th : pool) {
        th.join();
    }
    if (seconds != nullptr) {
        *seconds = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    }
    return failed ? make_error(first_error) : success();
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

extern "C" Error_t
vsag_index_search_buckets(vsag_index_t index, const float* queries, uint64_t nq, uint64_t dim, int64_t k,
                          const char* parameters, const int64_t* bucket_ids, const uint64_t* bucket_offsets, int64_t* ids,
                          float* dists, int64_t* result_dim) {
    auto* vi = static_cast<VsagIndex*>(index);
    if (vi == nullptr) {
        return make_error(VSAG_UNKNOWN_ERROR, "index is NULL");
    }
    if (ids == nullptr || dists == nullptr) {
        return make_error(VSAG_INVALID_ARGUMENT, "result arrays are NULL");
    }
    vsag::SearchRequest request;
    request.query_ = vsag::Dataset::Make();
    request.query_->Owner(false)
        ->Dim(static_cast<int64_t>(dim))
        ->NumElements(static_cast<int64_t>(nq))
        ->Float32Vectors(queries);
    request.topk_ = k;
    request.params_str_ = parameters ? parameters : "";
    if (bucket_offsets != nullptr && bucket_ids != nullptr) {
        request.bucket_ids_.resize(nq);
        for (uint64_t i = 0; i < nq; ++i) {
            request.bucket_ids_[i].assign(bucket_ids + bucket_offsets[i], bucket_ids + bucket_offsets[i + 1]);
        }
    }
    auto result = vi->index_->SearchWithRequest(request);
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

extern "C" Error_t
vsag_index_train(vsag_index_t index, const float* data, const int64_t* ids, uint64_t dim, uint64_t count) {
    auto* vi = static_cast<VsagIndex*>(index);
    if (vi == nullptr) {
        return make_error(VSAG_UNKNOWN_ERROR, "index is NULL");
    }
    auto result = vi->index_->Train(base_dataset(data, ids, dim, count));
    return result.has_value() ? success() : make_error(result.error());
}

extern "C" Error_t
vsag_index_calculate_distance_by_ids(vsag_index_t index, const float* query, uint64_t dim, const int64_t* ids,
                                     uint64_t count, float* dists) {
    return vsag_index_calculate_distances(index, query, 1, dim, ids, count, true, -1, nullptr, dists);
}

extern "C" Error_t
vsag_index_calculate_distances(vsag_index_t index, const float* queries, uint64_t nq, uint64_t dim, const int64_t* ids,
                               uint64_t count, bool precise, int64_t topk, int64_t* out_ids, float* out_dists) {
    auto* vi = static_cast<VsagIndex*>(index);
    if (vi == nullptr) {
        return make_error(VSAG_UNKNOWN_ERROR, "index is NULL");
    }
    if (out_dists == nullptr && count > 0) {
        return make_error(VSAG_INVALID_ARGUMENT, "output array is NULL");
    }
    auto q = vsag::Dataset::Make();
    q->Owner(false)->Dim(static_cast<int64_t>(dim))->NumElements(static_cast<int64_t>(nq))->Float32Vectors(queries);
    auto result = vi->index_->CalDistanceById(q, ids, static_cast<int64_t>(count), precise, topk);
    if (!result.has_value()) {
        return make_error(result.error());
    }
    const auto& r = result.value();
    const int64_t total = r->GetNumElements() * r->GetDim();
    if (total > 0) {
        std::memcpy(out_dists, r->GetDistances(), static_cast<size_t>(total) * sizeof(float));
        if (out_ids != nullptr && r->GetIds() != nullptr) {
            std::memcpy(out_ids, r->GetIds(), static_cast<size_t>(total) * sizeof(int64_t));
        }
    }
    return success();
}

extern "C" Error_t
vsag_search_result_enable_statistics(SearchResult_t* search_result) {
    if (search_result == nullptr) {
        return make_error(VSAG_UNKNOWN_ERROR, "search result is NULL");
    }
    std::lock_guard<std::mutex> lock(statistics_mutex);
    if (statistics_requests.count(search_result) != 0 || statistics_results.count(search_result) != 0) {
        return make_error(VSAG_UNKNOWN_ERROR, "search result statistics are already enabled");
    }
    statistics_requests.insert(search_result);
    return success();
}

extern "C" const char*
vsag_search_result_get_statistics(const SearchResult_t* search_result) {
    std::lock_guard<std::mutex> lock(statistics_mutex);
    auto it = statistics_results.find(search_result);
    return it == statistics_results.end() ? nullptr : it->second->c_str();
}

extern "C" void
vsag_search_result_destroy_statistics(SearchResult_t* search_result) {
    std::lock_guard<std::mutex> lock(statistics_mutex);
    statistics_requests.erase(search_result);
    statistics_results.erase(search_result);
}

extern "C" Error_t
vsag_serialize_file(vsag_index_t index, const char* file_path) {
    auto* vi = static_cast<VsagIndex*>(index);
    if (vi == nullptr || file_path == nullptr) {
        return make_error(VSAG_UNKNOWN_ERROR, "index or file path is NULL");
    }
    std::ofstream file(file_path, std::ios::binary | std::ios::trunc);
    if (!file.is_open()) {
        return make_error(VSAG_INTERNAL_ERROR, std::string("failed to open file for writing: ") + file_path);
    }
    auto result = vi->index_->Serialize(file);
    file.close();
    if (!result.has_value()) {
        return make_error(result.error());
    }
    if (file.fail()) {
        // a write or the closing flush did not reach the file (a full disk): the file is truncated
        return make_error(VSAG_INTERNAL_ERROR, std::string("failed to write file: ") + file_path);
    }
    return success();
}

extern "C" Error_t
vsag_deserialize_file(vsag_index_t index, const char* file_path) {
    auto* vi = static_cast<VsagIndex*>(index);
    if (vi == nullptr || file_path == nullptr) {
        return make_error(VSAG_UNKNOWN_ERROR, "index or file path is NULL");
    }
    std::ifstream file(file_path, std::ios::binary);
    if (!file.is_open()) {
        return make_error(VSAG_MISSING_FILE, std::string("failed to open file for reading: ") + file_path);
    }
    auto result = vi->index_->Deserialize(file);
    return result.has_value() ? success() : make_error(result.error());
}
