// Host-side mirror of the part of VSAG's public API that drives the search core:
//   vsag::Factory::CreateIndex("brute_force" | "ivf", json)  (include/vsag/factory.h:47-50)
//   vsag::Index::{Build, Add, KnnSearch, GetNumElements}       (include/vsag/index.h:126,150,284-374)
//   vsag::Dataset builder                                       (include/vsag/dataset.h:134-511)
//   vsag::Error / ErrorType                                     (include/vsag/errors.h:26-56)
//   vsag::Bitset, vsag::Filter                                  (include/vsag/bitset.h:27-101, filter.h:24-80)
// Same names, argument meaning, JSON keys and error behaviour; the arithmetic behind it runs in the HIP
// library (include/vsag_amd.h).  The reference returns tl::expected<T, Error>; Expected<T> below has the
// same has_value() / value() / error() surface.
#pragma once

#include <cstdint>
#include <functional>
#include <iosfwd>
#include <memory>
#include <string>
#include <utility>
#include <vector>

// The classes live in an inline namespace: source code says vsag::Index as with the reference, while the symbols
// (vsag::amd_gpu::Index ...) differ from the reference's, so that a program may link this library beside the real
// libvsag (one translation unit includes one of the two headers).
namespace vsag {
inline namespace amd_gpu {

#define VSAG_HOST_EXPORT __attribute__((visibility("default")))

enum class ErrorType {
    UNKNOWN_ERROR = 1,
    INTERNAL_ERROR,
    INVALID_ARGUMENT,
    WRONG_STATUS,
    BUILD_TWICE,
    INDEX_NOT_EMPTY,
    UNSUPPORTED_INDEX,
    UNSUPPORTED_INDEX_OPERATION,
    DIMENSION_NOT_EQUAL,
    INDEX_EMPTY,
    NO_ENOUGH_MEMORY,
    READ_ERROR,
    MISSING_FILE,
    INVALID_BINARY,
};

struct Error {
    Error(ErrorType t, std::string msg) : type(t), message(std::move(msg)) {
    }
    ErrorType type;
    std::string message;
};

template <typename T>
class Expected {
public:
    Expected(T value) : has_(true), value_(std::move(value)), error_(ErrorType::UNKNOWN_ERROR, "") {
    }
    Expected(Error error) : has_(false), value_(), error_(std::move(error)) {
    }
    bool
    has_value() const {
        return has_;
    }
    explicit operator bool() const {
        return has_;
    }
    T&
    value() {
        return value_;
    }
    const T&
    value() const {
        return value_;
    }
    T&
    operator*() {
        return value_;
    }
    T*
    operator->() {
        return &value_;
    }
    const Error&
    error() const {
        return error_;
    }

private:
    bool has_;
    T value_;
    Error error_;
};

// The reference's tl::expected<void, Error> of Train and the like.
template <>
class Expected<void> {
public:
    Expected() : has_(true), error_(ErrorType::UNKNOWN_ERROR, "") {
    }
    Expected(Error error) : has_(false), error_(std::move(error)) {
    }
    bool
    has_value() const {
        return has_;
    }
    explicit operator bool() const {
        return has_;
    }
    const Error&
    error() const {
        return error_;
    }

private:
    bool has_;
    Error error_;
};

// include/vsag/allocator.h:34-96: the caller's memory management.  An index created with an allocator takes the arrays
// of its results (ids, distances) from it; the dataset that owns them gives them back to it.  Device memory is not the
// allocator's business.
class Allocator {
public:
    virtual ~Allocator() = default;
    virtual std::string
    Name() = 0;
    virtual void*
    Allocate(uint64_t size) = 0;
    virtual void
    Deallocate(void* p) = 0;
    virtual void*
    Reallocate(void* p, uint64_t size) = 0;
};

class Dataset;
using DatasetPtr = std::shared_ptr<Dataset>;

// Column container with the reference's builder style.  An owning dataset frees ids / distances / vectors when it
// dies (results of a search are owning): through its allocator when it was given one (Owner(true, allocator),
// include/vsag/dataset.h:140-147), else with delete[].
class VSAG_HOST_EXPORT Dataset : public std::enable_shared_from_this<Dataset> {
public:
    static DatasetPtr
    Make() {
        return DatasetPtr(new Dataset());
    }
    ~Dataset() {
        if (owner_ && allocator_ != nullptr) {
            allocator_->Deallocate(const_cast<int64_t*>(ids_));
            allocator_->Deallocate(const_cast<float*>(distances_));
            allocator_->Deallocate(const_cast<float*>(vectors_));
        } else if (owner_) {
            delete[] ids_;
            delete[] distances_;
            delete[] vectors_;
        }
    }
    DatasetPtr
    Owner(bool is_owner, Allocator* allocator = nullptr) {
        owner_ = is_owner;
        allocator_ = allocator;
        return shared_from_this();
    }
    DatasetPtr
    NumElements(int64_t n) {
        num_elements_ = n;
        return shared_from_this();
    }
    DatasetPtr
    Dim(int64_t d) {
        dim_ = d;
        return shared_from_this();
    }
    DatasetPtr
    Ids(const int64_t* ids) {
        ids_ = ids;
        return shared_from_this();
    }
    DatasetPtr
    Distances(const float* d) {
        distances_ = d;
        return shared_from_this();
    }
    DatasetPtr
    Float32Vectors(const float* v) {
        vectors_ = v;
        return shared_from_this();
    }
    DatasetPtr
    Statistics(std::string s) {
        statistics_ = std::move(s);
        return shared_from_this();
    }
    int64_t
    GetNumElements() const {
        return num_elements_;
    }
    int64_t
    GetDim() const {
        return dim_;
    }
    const int64_t*
    GetIds() const {
        return ids_;
    }
    const float*
    GetDistances() const {
        return distances_;
    }
    const float*
    GetFloat32Vectors() const {
        return vectors_;
    }
    const std::string&
    GetStatistics() const {
        return statistics_;
    }

private:
    Dataset() = default;
    bool owner_ = true;
    Allocator* allocator_ = nullptr;
    int64_t num_elements_ = 0;
    int64_t dim_ = 0;
    const int64_t* ids_ = nullptr;
    const float* distances_ = nullptr;
    const float* vectors_ = nullptr;
    std::string statistics_;
};

// Pre-filter by bit mask: bit (label & 0xFFFFFFFF) set = the vector with that label is filtered OUT
// (BlackListFilter::CheckValid, src/impl/filter/black_list_filter.cpp:24-31).
class Bitset;
using BitsetPtr = std::shared_ptr<Bitset>;
class VSAG_HOST_EXPORT Bitset {
public:
    static BitsetPtr
    Make() {
        return BitsetPtr(new Bitset());
    }
    void
    Set(int64_t pos, bool value = true) {
        auto word = static_cast<size_t>(pos >> 6);
        if (word >= words_.size()) {
            if (!value) {
                return;
            }
            words_.resize(word + 1, 0);
        }
        const uint64_t bit = 1ULL << (pos & 63);
        words_[word] = value ? words_[word] | bit : words_[word] & ~bit;
    }
    bool
    Test(int64_t pos) const {
        auto word = static_cast<size_t>(pos >> 6);
        return word < words_.size() && ((words_[word] >> (pos & 63)) & 1ULL) != 0;
    }
    uint64_t
    Count() const {
        uint64_t c = 0;
        for (uint64_t w : words_) {
            c += static_cast<uint64_t>(__builtin_popcountll(w));
        }
        return c;
    }

private:
    Bitset() = default;
    std::vector<uint64_t> words_;
};

// Pre-filter by callback object: CheckValid(label) == true keeps the vector.
class Filter {
public:
    virtual ~Filter() = default;
    virtual bool
    CheckValid(int64_t id) const = 0;
};
using FilterPtr = std::shared_ptr<Filter>;

// include/vsag/search_request.h:34-230, the fields the brute_force and ivf indexes read.
enum class SearchMode {
    KNN_SEARCH = 1,
    RANGE_SEARCH = 2,
};

class SearchRequest {
public:
    DatasetPtr query_{nullptr};
    SearchMode mode_{SearchMode::KNN_SEARCH};
    int64_t topk_{10};
    float radius_{0.5F};
    int64_t limited_size_{-1};
    std::string params_str_{};
    bool enable_filter_{false};
    FilterPtr filter_{nullptr};
    bool enable_bitset_filter_{false};
    BitsetPtr bitset_filter_{nullptr};
    // ivf: the buckets every query scans, in scan order, instead of the routed ones (one list per query; empty =
    // default routing).  The hook by which a caller injects its own routing (ivf.cpp:2075-2112).
    std::vector<std::vector<int64_t>> bucket_ids_{};
};

class VSAG_HOST_EXPORT Index {
public:
    virtual ~Index() = default;

    // Trains the quantizers (and, for ivf, the partition) without inserting anything (include/vsag/index.h:150).
    virtual Expected<void>
    Train(const DatasetPtr& data) = 0;

    // include/vsag/index.h:333: the search described by `request` (filters are ANDed).
    virtual Expected<DatasetPtr>
    SearchWithRequest(const SearchRequest& request) const = 0;

    // include/vsag/index.h:575-633: distances between the query and the vectors with the given labels; -1 for a label
    // the index does not hold.  topk == -1: Dim = count, distances in the order of `ids`, no ids; topk > 0: the
    // min(topk, count) smallest, ascending, with their labels, unknown labels last.  calculate_precise_distance uses
    // the reorder vectors of an ivf index built with use_reorder, else the base codes.
    virtual Expected<DatasetPtr>
    CalDistanceById(const float* query, const int64_t* ids, int64_t count, bool calculate_precise_distance = true,
                    int64_t topk = -1) const = 0;
    virtual Expected<DatasetPtr>
    CalDistanceById(const DatasetPtr& query, const int64_t* ids, int64_t count, bool calculate_precise_distance = true,
                    int64_t topk = -1) const = 0;

    // include/vsag/index.h:903-940: the index as one stream (cells of codes, quantizer state and labels in the layout
    // of the reference, a footer with basic_info at the end) and back; Deserialize wants an empty index and a seekable
    // stream.
    virtual Expected<void>
    Serialize(std::ostream& out) const = 0;
    virtual Expected<void>
    Deserialize(std::istream& in) = 0;

    // Train + Add.  Returns the ids that could not be inserted (duplicates of ids already present).
    virtual Expected<std::vector<int64_t>>
    Build(const DatasetPtr& base) = 0;

    virtual Expected<std::vector<int64_t>>
    Add(const DatasetPtr& base) = 0;

    // query: NumElements rows of Dim floats.  One row -> result NumElements(1), Dim(count <= k), ascending
    // distances, ids are the user labels.  Several rows -> NumElements(nq), Dim(k), short rows padded with
    // id -1 / distance +inf (the batch convention of IVF::SearchWithRequest, src/algorithm/ivf/ivf.cpp:2137-2210).
    virtual Expected<DatasetPtr>
    KnnSearch(const DatasetPtr& query, int64_t k, const std::string& parameters) const = 0;

    // Pre-filtered searches (include/vsag/index.h:284-322).  invalid: see Bitset.  filter(label) == true
    // filters the vector OUT (BlackListFilter); a FilterPtr keeps what CheckValid accepts.
    virtual Expected<DatasetPtr>
    KnnSearch(const DatasetPtr& query, int64_t k, const std::string& parameters, BitsetPtr invalid) const = 0;
    virtual Expected<DatasetPtr>
    KnnSearch(const DatasetPtr& query, int64_t k, const std::string& parameters,
              const std::function<bool(int64_t)>& filter) const = 0;
    virtual Expected<DatasetPtr>
    KnnSearch(const DatasetPtr& query, int64_t k, const std::string& parameters, const FilterPtr& filter) const = 0;

    // Everything within `radius` (distance <= radius), ascending; limited_size > 0 keeps the nearest
    // limited_size, -1 keeps all, 0 is INVALID_ARGUMENT (include/vsag/index.h:394-466).
    virtual Expected<DatasetPtr>
    RangeSearch(const DatasetPtr& query, float radius, const std::string& parameters,
                int64_t limited_size = -1) const = 0;
    virtual Expected<DatasetPtr>
    RangeSearch(const DatasetPtr& query, float radius, const std::string& parameters, BitsetPtr invalid,
                int64_t limited_size = -1) const = 0;
    virtual Expected<DatasetPtr>
    RangeSearch(const DatasetPtr& query, float radius, const std::string& parameters,
                const std::function<bool(int64_t)>& filter, int64_t limited_size = -1) const = 0;
    virtual Expected<DatasetPtr>
    RangeSearch(const DatasetPtr& query, float radius, const std::string& parameters, const FilterPtr& filter,
                int64_t limited_size = -1) const = 0;

    virtual int64_t
    GetNumElements() const = 0;
};

class VSAG_HOST_EXPORT Factory {
public:
    // name: "brute_force" or "ivf".  parameters: {"dtype":"float32","metric_type":"l2"|"ip"|"cosine","dim":N,
    // "index_param":{...}} with the reference's keys (src/constants.cpp:195-216,255-265); unknown index_param
    // keys are INVALID_ARGUMENT "invalid config param: <key>" (src/utils/util_functions.cpp:45-66).
    // allocator (include/vsag/factory.h:47-50): where the index takes the host arrays of its results from; nullptr =
    // new[] / delete[].  It must outlive the index and every result the index returned.
    static Expected<std::shared_ptr<Index>>
    CreateIndex(const std::string& name, const std::string& parameters, Allocator* allocator = nullptr);
};

}  // namespace amd_gpu
}  // namespace vsag
