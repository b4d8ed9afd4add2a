// brute_force and ivf index classes on top of the HIP library: the host side of
//   BruteForce  (src/algorithm/bruteforce/bruteforce.cpp:91-95,213-293,354-635,1142-1376)
//   IVF         (src/algorithm/ivf/ivf.cpp:78-410,548-724,892-907,1565-1587,2052-2354)
//   Factory / Engine / IndexImpl error mapping (src/factory/engine.cpp:49-68, src/index/index_impl.h:309-322)
// It owns parameter parsing, the label table, Dataset packing and error mapping; every distance, every
// code and every centroid is computed by libvsag_amd.so.  There is no host arithmetic to fall back to.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <functional>
#include <limits>
#include <mutex>
#include <random>
#include <set>
#include <stdexcept>
#include <unordered_set>

#include "../../include/vsag_amd.h"
#include "json.h"
#include "vsag_host.h"

namespace vsag {
namespace {

using vsag_host::Json;

struct VsagException : public std::exception {
    VsagException(ErrorType t, std::string m) : type(t), message(std::move(m)) {
    }
    const char*
    what() const noexcept override {
        return message.c_str();
    }
    ErrorType type;
    std::string message;
};

#define CHECK_ARGUMENT(cond, msg)                                        \
    do {                                                                 \
        if (!(cond)) {                                                   \
            throw VsagException(ErrorType::INVALID_ARGUMENT, (msg));     \
        }                                                                \
    } while (0)

// Device call: 0 or throw with the library's message, mapped like src/common.h:23-35 maps exceptions.
void
dev(int rc) {
    if (rc == 0) {
        return;
    }
    ErrorType t = ErrorType::INTERNAL_ERROR;
    if (rc == VSAG_AMD_INVALID_ARGUMENT) {
        t = ErrorType::INVALID_ARGUMENT;
    } else if (rc == VSAG_AMD_NO_ENOUGH_MEMORY) {
        t = ErrorType::NO_ENOUGH_MEMORY;
    }
    throw VsagException(t, vsag_amd_last_error());
}

// SAFE_CALL of the reference (src/common.h:23-35).
template <typename T, typename F>
Expected<T>
safe_call(F&& f) {
    try {
        return Expected<T>(f());
    } catch (const VsagException& e) {
        return Expected<T>(Error(e.type, e.message));
    } catch (const std::bad_alloc&) {
        return Expected<T>(Error(ErrorType::NO_ENOUGH_MEMORY, "not enough memory"));
    } catch (const std::invalid_argument& e) {
        return Expected<T>(Error(ErrorType::INVALID_ARGUMENT, e.what()));
    } catch (const std::exception& e) {
        return Expected<T>(Error(ErrorType::UNKNOWN_ERROR, e.what()));
    }
}

struct DevBuf {
    void* p = nullptr;
    size_t bytes = 0;
    DevBuf() = default;
    DevBuf(const DevBuf&) = delete;
    DevBuf&
    operator=(const DevBuf&) = delete;
    ~DevBuf() {
        release();
    }
    void
    release() {
        if (p != nullptr) {
            vsag_amd_free(p);
            p = nullptr;
            bytes = 0;
        }
    }
    // Contents are not kept.
    void
    reserve(size_t n) {
        if (n <= bytes) {
            return;
        }
        release();
        dev(vsag_amd_malloc(&p, n));
        bytes = n;
    }
    // Keeps the first `keep` bytes.
    void
    grow(size_t n, size_t keep) {
        if (n <= bytes) {
            return;
        }
        size_t cap = std::max(n, bytes + bytes / 2);
        void* q = nullptr;
        dev(vsag_amd_malloc(&q, cap));
        if (keep > 0) {
            dev(vsag_amd_memcpy_d2d(q, p, keep, nullptr));
            dev(vsag_amd_stream_synchronize(nullptr));
        }
        if (p != nullptr) {
            vsag_amd_free(p);
        }
        p = q;
        bytes = cap;
    }
    template <typename T>
    T*
    as() const {
        return static_cast<T*>(p);
    }
};

struct CommonParam {
    int metric = VSAG_AMD_METRIC_L2;
    uint32_t dim = 0;
};

// IndexCommonParam::CheckAndCreate (src/index_common_param.cpp:117-174).
CommonParam
parse_common(const Json& params) {
    CHECK_ARGUMENT(params.IsObject(), "parameters must be a JSON object");
    CHECK_ARGUMENT(params.Contains("dtype"), "parameters must contains dtype");
    const std::string dtype = params["dtype"].GetString();
    CHECK_ARGUMENT(dtype == "float32", "parameters[dtype] must be float32 for this index, got " + dtype);
    CHECK_ARGUMENT(params.Contains("metric_type"), "parameters must contains metric_type");
    const std::string metric = params["metric_type"].GetString();
    CommonParam c;
    if (metric == "l2") {
        c.metric = VSAG_AMD_METRIC_L2;
    } else if (metric == "ip") {
        c.metric = VSAG_AMD_METRIC_IP;
    } else if (metric == "cosine") {
        c.metric = VSAG_AMD_METRIC_COSINE;
    } else {
        throw VsagException(ErrorType::INVALID_ARGUMENT,
                            "parameters[metric_type] must in [l2, ip, cosine], now is " + metric);
    }
    CHECK_ARGUMENT(params.Contains("dim"), "parameters must contain dim");
    int64_t dim = params["dim"].GetInt();
    CHECK_ARGUMENT(dim > 0 && dim <= 65536, "parameters[dim] must be in [1, 65536], got " + std::to_string(dim));
    c.dim = static_cast<uint32_t>(dim);
    return c;
}

int
kind_from_name(const std::string& name) {
    static const std::pair<const char*, int> kinds[] = {
        {"fp32", VSAG_AMD_KIND_FP32}, {"sq8", VSAG_AMD_KIND_SQ8}, {"sq4", VSAG_AMD_KIND_SQ4},
        {"sq4_uniform", VSAG_AMD_KIND_SQ4_UNIFORM}, {"sq8_uniform", VSAG_AMD_KIND_SQ8_UNIFORM},
        {"rabitq", VSAG_AMD_KIND_RABITQ}};
    for (const auto& k : kinds) {
        if (name == k.first) {
            return k.second;
        }
    }
    throw VsagException(ErrorType::INVALID_ARGUMENT, "unsupported quantization type on the GPU path: " + name);
}

// Quantizer state on the device (the Quantizer<Q> objects of src/quantization/).
struct Quantizer {
    int kind = VSAG_AMD_KIND_FP32;
    int metric = VSAG_AMD_METRIC_L2;
    uint32_t dim = 0;
    int rabitq_query_bits = 32;
    bool trained = false;
    DevBuf lb, diff, bounds, rotation, centroid;

    uint64_t
    code_size() const {
        return vsag_amd_code_size(kind, metric, dim, rabitq_query_bits);
    }

    // Random orthogonal matrix: Gram-Schmidt on a Gaussian matrix (the reference takes the Q of a LAPACK QR,
    // src/impl/transform/random_orthogonal_transformer.cpp:97-148, from std::random_device; here the seed is
    // fixed so that a build is reproducible).
    static std::vector<float>
    random_rotation(uint32_t d, uint32_t seed) {
        std::mt19937 gen(seed);
        std::normal_distribution<double> nd(0.0, 1.0);
        std::vector<double> m(static_cast<size_t>(d) * d);
        for (auto& v : m) {
            v = nd(gen);
        }
        for (uint32_t i = 0; i < d; ++i) {
            double* r = m.data() + static_cast<size_t>(i) * d;
            for (int pass = 0; pass < 2; ++pass) {
                for (uint32_t j = 0; j < i; ++j) {
                    const double* q = m.data() + static_cast<size_t>(j) * d;
                    double dot = 0;
                    for (uint32_t c = 0; c < d; ++c) {
                        dot += r[c] * q[c];
                    }
                    for (uint32_t c = 0; c < d; ++c) {
                        r[c] -= dot * q[c];
                    }
                }
            }
            double n = 0;
            for (uint32_t c = 0; c < d; ++c) {
                n += r[c] * r[c];
            }
            n = std::sqrt(n);
            for (uint32_t c = 0; c < d; ++c) {
                r[c] /= n;
            }
        }
        return std::vector<float>(m.begin(), m.end());
    }

    void
    train(const float* x_dev, uint64_t n) {
        if (trained || n == 0) {
            return;
        }
        DevBuf ws;
        switch (kind) {
            case VSAG_AMD_KIND_FP32:
                break;
            case VSAG_AMD_KIND_SQ8:
            case VSAG_AMD_KIND_SQ4: {
                // ScalarQuantizer::TrainImpl: TRUNC_BOUND, default sample (scalar_quantizer.cpp:52-73).
                lb.reserve(dim * 4);
                diff.reserve(dim * 4);
                size_t wsb = vsag_amd_sq_train_workspace_bytes(n, dim, 0);
                ws.reserve(wsb);
                dev(vsag_amd_sq_train(x_dev, n, dim, kind == VSAG_AMD_KIND_SQ8 ? 8 : 4, metric,
                                      VSAG_AMD_SQ_TRAIN_TRUNC_BOUND, 0.05F, 0, lb.as<float>(), diff.as<float>(), ws.p,
                                      wsb, nullptr));
                break;
            }
            case VSAG_AMD_KIND_SQ4_UNIFORM:
            case VSAG_AMD_KIND_SQ8_UNIFORM: {
                // sq4_uniform: TRUNC_BOUND with trunc_rate 0.05 (not user-settable for these indexes);
                // sq8_uniform: CLASSIC (sq4_uniform_quantizer.cpp:101-103, sq8_uniform_quantizer.cpp:89-91).
                bounds.reserve(8);
                size_t wsb = vsag_amd_sq_train_workspace_bytes(n, dim, 0);
                ws.reserve(wsb);
                bool four = kind == VSAG_AMD_KIND_SQ4_UNIFORM;
                dev(vsag_amd_sq_train_uniform(x_dev, n, dim, four ? 4 : 8, metric,
                                              four ? VSAG_AMD_SQ_TRAIN_TRUNC_BOUND : VSAG_AMD_SQ_TRAIN_CLASSIC, 0.05F,
                                              0, bounds.as<float>(), ws.p, wsb, nullptr));
                break;
            }
            case VSAG_AMD_KIND_RABITQ: {
                std::vector<float> rot = random_rotation(dim, 20240229U);
                rotation.reserve(rot.size() * 4);
                centroid.reserve(dim * 4);
                dev(vsag_amd_memcpy_h2d(rotation.p, rot.data(), rot.size() * 4, nullptr));
                dev(vsag_amd_rabitq_train(x_dev, n, dim, rotation.as<float>(), centroid.as<float>(), nullptr));
                break;
            }
        }
        dev(vsag_amd_stream_synchronize(nullptr));
        trained = true;
    }

    // Codes in the reference layout, n x code_size, into `codes` (device).  fp32 needs no encoding.
    void
    encode(const float* x_dev, uint64_t n, uint8_t* codes) const {
        switch (kind) {
            case VSAG_AMD_KIND_FP32:
                break;
            case VSAG_AMD_KIND_SQ8:
            case VSAG_AMD_KIND_SQ4:
                dev(vsag_amd_sq_encode(x_dev, n, dim, kind == VSAG_AMD_KIND_SQ8 ? 8 : 4, metric, lb.as<float>(),
                                       diff.as<float>(), codes, nullptr));
                break;
            case VSAG_AMD_KIND_SQ4_UNIFORM:
            case VSAG_AMD_KIND_SQ8_UNIFORM:
                dev(vsag_amd_squ_encode(x_dev, n, dim, kind == VSAG_AMD_KIND_SQ4_UNIFORM ? 4 : 8, metric,
                                        bounds.as<float>(), codes, nullptr));
                break;
            case VSAG_AMD_KIND_RABITQ:
                dev(vsag_amd_rabitq_encode(x_dev, n, dim, rotation.as<float>(), centroid.as<float>(), metric,
                                           rabitq_query_bits, codes, nullptr));
                break;
        }
    }

    vsag_amd_store_t*
    make_store() const {
        vsag_amd_store_params_t p{};
        p.kind = kind;
        p.metric = metric;
        p.dim = dim;
        p.rabitq_query_bits = rabitq_query_bits;
        if (kind == VSAG_AMD_KIND_SQ8 || kind == VSAG_AMD_KIND_SQ4) {
            p.lower_bound_dev = lb.as<float>();
            p.diff_dev = diff.as<float>();
        } else if (kind == VSAG_AMD_KIND_SQ4_UNIFORM || kind == VSAG_AMD_KIND_SQ8_UNIFORM) {
            p.lower_bound_dev = bounds.as<float>();
        } else if (kind == VSAG_AMD_KIND_RABITQ) {
            p.rotation_dev = rotation.as<float>();
            p.centroid_dev = centroid.as<float>();
        }
        vsag_amd_store_t* s = nullptr;
        dev(vsag_amd_store_create(&p, &s));
        return s;
    }
};

struct StoreHandle {
    vsag_amd_store_t* s = nullptr;
    ~StoreHandle() {
        if (s != nullptr) {
            vsag_amd_store_destroy(s);
        }
    }
};

void
check_base(const DatasetPtr& base, uint32_t dim) {
    CHECK_ARGUMENT(base != nullptr, "base dataset is null");
    CHECK_ARGUMENT(base->GetNumElements() >= 0, "number of elements must not be negative");
    if (base->GetNumElements() == 0) {
        return;
    }
    CHECK_ARGUMENT(base->GetDim() == static_cast<int64_t>(dim),
                   "base.dim(" + std::to_string(base->GetDim()) + ") must be equal to index.dim(" +
                       std::to_string(dim) + ")");
    CHECK_ARGUMENT(base->GetFloat32Vectors() != nullptr, "base.float_vector is nullptr");
    CHECK_ARGUMENT(base->GetIds() != nullptr, "base.ids is nullptr");
}

void
check_query(const DatasetPtr& query, int64_t k, uint32_t dim) {
    CHECK_ARGUMENT(query != nullptr, "query dataset is null");
    CHECK_ARGUMENT(k > 0, "k(" + std::to_string(k) + ") must be greater than 0");
    CHECK_ARGUMENT(query->GetNumElements() >= 1, "query dataset should contain at least 1 vector");
    CHECK_ARGUMENT(query->GetDim() == static_cast<int64_t>(dim),
                   "query.dim(" + std::to_string(query->GetDim()) + ") must be equal to index.dim(" +
                       std::to_string(dim) + ")");
    CHECK_ARGUMENT(query->GetFloat32Vectors() != nullptr, "query.float_vector is nullptr");
}

// pack_knn_result (src/algorithm/inner_index_interface.cpp:1133-1147) for one query, and the padded batch
// form of IVF::SearchWithRequest (ivf.cpp:2137-2210) for several.
DatasetPtr
pack_results(const std::vector<uint32_t>& ids, const std::vector<float>& dists, int64_t nq, int64_t k,
             const std::vector<int64_t>& labels, const std::string& stats) {
    for (int64_t i = 0; i < nq * k; ++i) {
        if (ids[i] != VSAG_AMD_INVALID_ID && ids[i] >= labels.size()) {
            throw VsagException(ErrorType::INTERNAL_ERROR,
                                "search returned inner id " + std::to_string(ids[i]) + " of " + std::to_string(labels.size()));
        }
    }
    auto result = Dataset::Make();
    if (nq == 1) {
        int64_t count = 0;
        while (count < k && ids[count] != VSAG_AMD_INVALID_ID) {
            ++count;
        }
        auto* out_ids = new int64_t[std::max<int64_t>(count, 1)];
        auto* out_d = new float[std::max<int64_t>(count, 1)];
        for (int64_t i = 0; i < count; ++i) {
            out_ids[i] = labels[ids[i]];
            out_d[i] = dists[i];
        }
        result->NumElements(1)->Dim(count)->Ids(out_ids)->Distances(out_d)->Owner(true)->Statistics(stats);
        return result;
    }
    auto* out_ids = new int64_t[nq * k];
    auto* out_d = new float[nq * k];
    for (int64_t i = 0; i < nq * k; ++i) {
        if (ids[i] == VSAG_AMD_INVALID_ID) {
            out_ids[i] = -1;
            out_d[i] = std::numeric_limits<float>::infinity();
        } else {
            out_ids[i] = labels[ids[i]];
            out_d[i] = dists[i];
        }
    }
    result->NumElements(nq)->Dim(k)->Ids(out_ids)->Distances(out_d)->Owner(true)->Statistics(stats);
    return result;
}

// Ids of `base` that are already present (or repeated inside `base`): they are reported back and skipped,
// as BruteForce::Add / IVF::Add do through the label table.
std::vector<int64_t>
split_new_rows(const DatasetPtr& base, std::unordered_set<int64_t>& known, std::vector<int64_t>& rows) {
    std::vector<int64_t> failed;
    const int64_t* ids = base->GetIds();
    for (int64_t i = 0; i < base->GetNumElements(); ++i) {
        if (known.insert(ids[i]).second) {
            rows.push_back(i);
        } else {
            failed.push_back(ids[i]);
        }
    }
    return failed;
}

// Uploads the selected rows (all rows when nothing was skipped) as one n x dim device matrix.
void
upload_rows(const DatasetPtr& base, const std::vector<int64_t>& rows, uint32_t dim, DevBuf& out) {
    const float* src = base->GetFloat32Vectors();
    size_t row_bytes = static_cast<size_t>(dim) * 4;
    out.reserve(std::max<size_t>(rows.size() * row_bytes, 4));
    if (static_cast<int64_t>(rows.size()) == base->GetNumElements()) {
        dev(vsag_amd_memcpy_h2d(out.p, src, rows.size() * row_bytes, nullptr));
        return;
    }
    std::vector<float> staged(rows.size() * dim);
    for (size_t i = 0; i < rows.size(); ++i) {
        std::memcpy(staged.data() + i * dim, src + rows[i] * dim, row_bytes);
    }
    dev(vsag_amd_memcpy_h2d(out.p, staged.data(), staged.size() * 4, nullptr));
}

void
reject_unknown_keys(const Json& index_param, const std::set<std::string>& known) {
    for (const auto& m : index_param.members) {
        if (known.count(m.first) == 0) {
            throw VsagException(ErrorType::INVALID_ARGUMENT, "invalid config param: " + m.first);
        }
    }
}

// What a search asks for beyond (query, k): a pre-filter on labels and / or a radius.
struct SearchSpec {
    bool range = false;
    float radius = 0.0F;
    int64_t limited_size = -1;
    std::function<bool(int64_t)> valid;  // empty = every label is kept
};

// Deny mask over inner ids for the device scans (bit set = filtered out), kept on the host as well so that
// a range search can add the ids it has already returned.
struct DenyMask {
    std::vector<uint32_t> words;
    DevBuf dev_words;
    bool active = false;

    void
    init(const std::vector<int64_t>& labels, const std::function<bool(int64_t)>& valid, bool force) {
        active = static_cast<bool>(valid) || force;
        if (!active) {
            return;
        }
        words.assign((labels.size() + 31) / 32, 0U);
        if (valid) {
            for (size_t i = 0; i < labels.size(); ++i) {
                if (!valid(labels[i])) {
                    words[i >> 5] |= 1U << (i & 31);
                }
            }
        }
        upload();
    }
    void
    deny(uint32_t id) {
        words[id >> 5] |= 1U << (id & 31);
    }
    void
    upload() {
        dev_words.reserve(std::max<size_t>(words.size() * 4, 4));
        dev(vsag_amd_memcpy_h2d(dev_words.p, words.data(), words.size() * 4, nullptr));
    }
    vsag_amd_search_options_t
    options(const SearchSpec& spec, float radius_slack) const {
        vsag_amd_search_options_t o{};
        o.deny_bits_dev = active ? dev_words.as<uint32_t>() : nullptr;
        o.use_radius = spec.range ? 1 : 0;
        o.radius = spec.radius + radius_slack;
        return o;
    }
};

constexpr int64_t kMaxDeviceK = 1024;  // largest k of one device scan

// One ascending row of (distance, inner id) as a single-query result dataset.
DatasetPtr
pack_row(const std::vector<std::pair<float, uint32_t>>& row, const std::vector<int64_t>& labels,
         const std::string& stats) {
    std::vector<uint32_t> ids(std::max<size_t>(row.size(), 1), VSAG_AMD_INVALID_ID);
    std::vector<float> dists(ids.size(), std::numeric_limits<float>::infinity());
    for (size_t i = 0; i < row.size(); ++i) {
        dists[i] = row[i].first;
        ids[i] = row[i].second;
    }
    return pack_results(ids, dists, 1, static_cast<int64_t>(ids.size()), labels, stats);
}

// The search overloads of the public interface, reduced to one virtual search().
class GpuIndex : public Index {
public:
    Expected<DatasetPtr>
    KnnSearch(const DatasetPtr& query, int64_t k, const std::string& parameters) const override {
        return run(query, k, parameters, SearchSpec{});
    }
    Expected<DatasetPtr>
    KnnSearch(const DatasetPtr& query, int64_t k, const std::string& parameters, BitsetPtr invalid) const override {
        return run(query, k, parameters, with_bitset(SearchSpec{}, invalid));
    }
    Expected<DatasetPtr>
    KnnSearch(const DatasetPtr& query, int64_t k, const std::string& parameters,
              const std::function<bool(int64_t)>& filter) const override {
        return run(query, k, parameters, with_function(SearchSpec{}, filter));
    }
    Expected<DatasetPtr>
    KnnSearch(const DatasetPtr& query, int64_t k, const std::string& parameters,
              const FilterPtr& filter) const override {
        return run(query, k, parameters, with_filter(SearchSpec{}, filter));
    }
    Expected<DatasetPtr>
    RangeSearch(const DatasetPtr& query, float radius, const std::string& parameters,
                int64_t limited_size) const override {
        return run(query, 1, parameters, range_spec(radius, limited_size));
    }
    Expected<DatasetPtr>
    RangeSearch(const DatasetPtr& query, float radius, const std::string& parameters, BitsetPtr invalid,
                int64_t limited_size) const override {
        return run(query, 1, parameters, with_bitset(range_spec(radius, limited_size), invalid));
    }
    Expected<DatasetPtr>
    RangeSearch(const DatasetPtr& query, float radius, const std::string& parameters,
                const std::function<bool(int64_t)>& filter, int64_t limited_size) const override {
        return run(query, 1, parameters, with_function(range_spec(radius, limited_size), filter));
    }
    Expected<DatasetPtr>
    RangeSearch(const DatasetPtr& query, float radius, const std::string& parameters, const FilterPtr& filter,
                int64_t limited_size) const override {
        return run(query, 1, parameters, with_filter(range_spec(radius, limited_size), filter));
    }

protected:
    virtual DatasetPtr
    search(const DatasetPtr& query, int64_t k, const std::string& parameters, const SearchSpec& spec) const = 0;

private:
    Expected<DatasetPtr>
    run(const DatasetPtr& query, int64_t k, const std::string& parameters, const SearchSpec& spec) const {
        return safe_call<DatasetPtr>([&]() {
            if (spec.range) {
                // InnerIndexInterface::validate_range_args (inner_index_interface.cpp:1252-1259)
                CHECK_ARGUMENT(std::isfinite(spec.radius), "radius must be finite");
                CHECK_ARGUMENT(spec.radius >= 0.0F,
                               "radius(" + std::to_string(spec.radius) + ") must be greater equal than 0");
                CHECK_ARGUMENT(spec.limited_size != 0, "limited_size(0) must not be equal to 0");
            }
            return search(query, k, parameters, spec);
        });
    }
    static SearchSpec
    range_spec(float radius, int64_t limited_size) {
        SearchSpec s;
        s.range = true;
        s.radius = radius;
        s.limited_size = limited_size;
        return s;
    }
    static SearchSpec
    with_bitset(SearchSpec s, const BitsetPtr& invalid) {
        if (invalid != nullptr) {
            s.valid = [invalid](int64_t label) { return !invalid->Test(label & 0xFFFFFFFFLL); };
        }
        return s;
    }
    static SearchSpec
    with_function(SearchSpec s, const std::function<bool(int64_t)>& filter) {
        if (filter) {
            s.valid = [filter](int64_t label) { return !filter(label); };
        }
        return s;
    }
    static SearchSpec
    with_filter(SearchSpec s, const FilterPtr& filter) {
        if (filter != nullptr) {
            s.valid = [filter](int64_t label) { return filter->CheckValid(label); };
        }
        return s;
    }
};

// ------------------------------------------------------------------------------------------- brute_force
class BruteForce : public GpuIndex {
public:
    BruteForce(const CommonParam& common, const Json& index_param) {
        static const std::set<std::string> known = {
            "base_quantization_type", "base_io_type", "base_pq_dim", "base_file_path", "precise_quantization_type",
            "precise_io_type", "precise_file_path", "thread_count", "use_residual", "use_reorder",
            "use_attribute_filter", "rabitq_bits_per_dim_query", "rabitq_bits_per_dim_base", "rabitq_use_fht"};
        reject_unknown_keys(index_param, known);
        q_.metric = common.metric;
        q_.dim = common.dim;
        q_.kind = VSAG_AMD_KIND_FP32;
        if (index_param.Contains("base_quantization_type")) {
            q_.kind = kind_from_name(index_param["base_quantization_type"].GetString());
        }
        if (index_param.Contains("rabitq_bits_per_dim_query")) {
            q_.rabitq_query_bits = static_cast<int>(index_param["rabitq_bits_per_dim_query"].GetInt());
        }
        if (q_.kind == VSAG_AMD_KIND_RABITQ) {
            CHECK_ARGUMENT(q_.rabitq_query_bits == 4 || q_.rabitq_query_bits == 32,
                           "rabitq_bits_per_dim_query must be 4 or 32");
            if (index_param.Contains("rabitq_bits_per_dim_base")) {
                CHECK_ARGUMENT(index_param["rabitq_bits_per_dim_base"].GetInt() == 1,
                               "the GPU path supports rabitq_bits_per_dim_base = 1 only");
            }
            if (index_param.Contains("rabitq_use_fht")) {
                CHECK_ARGUMENT(!index_param["rabitq_use_fht"].GetBool(), "rabitq_use_fht is not supported");
            }
        }
    }

    Expected<std::vector<int64_t>>
    Build(const DatasetPtr& base) override {
        return safe_call<std::vector<int64_t>>([&]() {
            std::lock_guard<std::mutex> lock(mutex_);
            if (!labels_.empty()) {
                throw VsagException(ErrorType::BUILD_TWICE, "failed to build index: index is not empty");
            }
            return add_locked(base);
        });
    }

    Expected<std::vector<int64_t>>
    Add(const DatasetPtr& base) override {
        return safe_call<std::vector<int64_t>>([&]() {
            std::lock_guard<std::mutex> lock(mutex_);
            return add_locked(base);
        });
    }

protected:
    DatasetPtr
    search(const DatasetPtr& query, int64_t k, const std::string& parameters, const SearchSpec& spec) const override {
        check_query(query, k, q_.dim);
        if (!parameters.empty()) {
            Json p = Json::Parse(parameters);  // {"parallelism": p}, optionally under "brute_force"
            CHECK_ARGUMENT(p.IsObject(), "search parameters must be a JSON object");
        }
        std::lock_guard<std::mutex> lock(mutex_);
        const int64_t nq = query->GetNumElements();
        if (labels_.empty()) {
            auto empty = Dataset::Make();
            empty->NumElements(1)->Dim(0);
            return empty;
        }
        // One device scan returns at most 1024 results per query.  A range search, and a KnnSearch with a larger
        // k, run scan after scan for one query: what a scan returned is denied to the next one, so the rows come
        // out in ascending order.
        const bool looped = spec.range || k > kMaxDeviceK;
        CHECK_ARGUMENT(!looped || nq == 1, spec.range ? "range search takes one query"
                                                      : "k above 1024 is supported for one query per call");
        queries_.reserve(static_cast<size_t>(nq) * q_.dim * 4);
        dev(vsag_amd_memcpy_h2d(queries_.p, query->GetFloat32Vectors(), static_cast<size_t>(nq) * q_.dim * 4, nullptr));
        DenyMask mask;
        mask.init(labels_, spec.valid, looped);
        const vsag_amd_search_options_t opt = mask.options(spec, 0.0F);
        // distance_evaluations as the reference counts them: every stored vector once per query
        const std::string stats = "{\"dist_cmp\":" + std::to_string(labels_.size() * static_cast<size_t>(nq)) + "}";
        const auto n = static_cast<int64_t>(labels_.size());
        if (!looped) {
            const auto kk = static_cast<uint32_t>(k);
            std::vector<uint32_t> ids;
            std::vector<float> dists;
            scan(nq, kk, opt, ids, dists);
            return pack_results(ids, dists, nq, k, labels_, stats);
        }
        std::vector<std::pair<float, uint32_t>> row;
        int64_t remaining = spec.range ? (spec.limited_size > 0 ? spec.limited_size : n) : k;
        while (remaining > 0) {
            const auto kk = static_cast<uint32_t>(std::min<int64_t>({remaining, kMaxDeviceK, n}));
            std::vector<uint32_t> ids;
            std::vector<float> dists;
            scan(1, kk, opt, ids, dists);
            uint32_t got = 0;
            while (got < kk && ids[got] != VSAG_AMD_INVALID_ID) {
                row.emplace_back(dists[got], ids[got]);
                mask.deny(ids[got]);
                ++got;
            }
            remaining -= got;
            if (got < kk) {
                break;
            }
            mask.upload();
        }
        if (row.empty()) {
            auto empty = Dataset::Make();
            empty->NumElements(1)->Dim(0)->Statistics(stats);
            return empty;
        }
        return pack_row(row, labels_, stats);
    }

public:
    int64_t
    GetNumElements() const override {
        std::lock_guard<std::mutex> lock(mutex_);
        return static_cast<int64_t>(labels_.size());
    }

private:
    // One device scan of the uploaded queries; results copied to the host.
    void
    scan(int64_t nq, uint32_t kk, const vsag_amd_search_options_t& opt, std::vector<uint32_t>& ids,
         std::vector<float>& dists) const {
        out_ids_.reserve(static_cast<size_t>(nq) * kk * 4);
        out_d_.reserve(static_cast<size_t>(nq) * kk * 4);
        size_t wsb = vsag_amd_flat_scan_workspace_bytes(store_.s, nq, kk);
        workspace_.reserve(wsb);
        dev(vsag_amd_flat_scan_topk_ex(store_.s, queries_.as<float>(), nq, kk, &opt, out_ids_.as<uint32_t>(),
                                       out_d_.as<float>(), workspace_.p, wsb, nullptr));
        ids.resize(static_cast<size_t>(nq) * kk);
        dists.resize(ids.size());
        dev(vsag_amd_memcpy_d2h(ids.data(), out_ids_.p, ids.size() * 4, nullptr));
        dev(vsag_amd_memcpy_d2h(dists.data(), out_d_.p, dists.size() * 4, nullptr));
    }

    std::vector<int64_t>
    add_locked(const DatasetPtr& base) {
        check_base(base, q_.dim);
        std::vector<int64_t> rows;
        std::vector<int64_t> failed = split_new_rows(base, known_, rows);
        if (rows.empty()) {
            return failed;
        }
        DevBuf x;
        upload_rows(base, rows, q_.dim, x);
        q_.train(x.as<float>(), rows.size());
        if (store_.s == nullptr) {
            store_.s = q_.make_store();
        }
        if (q_.kind == VSAG_AMD_KIND_FP32) {
            dev(vsag_amd_store_append(store_.s, x.as<uint8_t>(), rows.size(), nullptr));
        } else {
            DevBuf codes;
            codes.reserve(rows.size() * q_.code_size());
            q_.encode(x.as<float>(), rows.size(), codes.as<uint8_t>());
            dev(vsag_amd_store_append(store_.s, codes.as<uint8_t>(), rows.size(), nullptr));
            dev(vsag_amd_stream_synchronize(nullptr));
        }
        dev(vsag_amd_stream_synchronize(nullptr));
        for (int64_t r : rows) {
            labels_.push_back(base->GetIds()[r]);
        }
        return failed;
    }

    Quantizer q_;
    StoreHandle store_;
    std::vector<int64_t> labels_;  // inner id -> label (LabelTable)
    std::unordered_set<int64_t> known_;
    mutable std::mutex mutex_;
    mutable DevBuf queries_, out_ids_, out_d_, workspace_;
};

// ------------------------------------------------------------------------------------------- ivf
class IVF : public GpuIndex {
public:
    IVF(const CommonParam& common, const Json& index_param) : common_(common) {
        static const std::set<std::string> known = {
            "buckets_count", "base_quantization_type", "base_io_type", "base_pq_dim", "base_file_path",
            "base_enable_read_cache", "base_cache_total_size", "precise_enable_read_cache",
            "precise_cache_total_size", "ivf_train_type", "use_reorder", "precise_quantization_type",
            "precise_io_type", "precise_file_path", "precise_codes_layout", "buckets_per_data", "use_residual",
            "thread_count", "train_sample_count", "use_attribute_filter", "partition_strategy_type",
            "rabitq_bits_per_dim_query", "rabitq_bits_per_dim_base", "rabitq_use_fht", "rabitq_version",
            "rabitq_error_rate", "fast_encode_rabitq", "fast_encode_rabitq_rounds", "graph_build_threshold"};
        reject_unknown_keys(index_param, known);
        q_.metric = common.metric;
        q_.dim = common.dim;
        if (index_param.Contains("base_quantization_type")) {
            q_.kind = kind_from_name(index_param["base_quantization_type"].GetString());
        }
        if (index_param.Contains("rabitq_bits_per_dim_query")) {
            q_.rabitq_query_bits = static_cast<int>(index_param["rabitq_bits_per_dim_query"].GetInt());
        }
        if (q_.kind == VSAG_AMD_KIND_RABITQ) {
            CHECK_ARGUMENT(q_.rabitq_query_bits == 4 || q_.rabitq_query_bits == 32,
                           "rabitq_bits_per_dim_query must be 4 or 32");
        }
        if (index_param.Contains("buckets_count")) {
            int64_t b = index_param["buckets_count"].GetInt();
            CHECK_ARGUMENT(b >= 1 && b <= (1 << 24), "buckets_count must be in [1, 2^24], got " + std::to_string(b));
            nlist_ = static_cast<uint32_t>(b);
        }
        if (index_param.Contains("use_reorder")) {
            use_reorder_ = index_param["use_reorder"].GetBool();
        }
        if (index_param.Contains("precise_quantization_type")) {
            CHECK_ARGUMENT(index_param["precise_quantization_type"].GetString() == "fp32",
                           "the GPU path reranks with precise_quantization_type = fp32 only");
        }
        if (index_param.Contains("ivf_train_type")) {
            const std::string t = index_param["ivf_train_type"].GetString();
            CHECK_ARGUMENT(t == "kmeans" || t == "random", "ivf_train_type must be kmeans or random, got " + t);
            train_random_ = t == "random";
        }
        if (index_param.Contains("buckets_per_data")) {
            CHECK_ARGUMENT(index_param["buckets_per_data"].GetInt() == 1,
                           "the GPU path supports buckets_per_data = 1 only");
        }
        if (index_param.Contains("use_residual")) {
            CHECK_ARGUMENT(!index_param["use_residual"].GetBool(), "the GPU path does not support use_residual");
        }
        if (index_param.Contains("partition_strategy_type")) {
            CHECK_ARGUMENT(index_param["partition_strategy_type"].GetString() == "ivf",
                           "the GPU path supports the nearest-centroid partition strategy only");
        }
        // ivf_parameter.cpp:88-98: default max(65536, 64 * buckets_count), at least 512.
        train_sample_count_ = std::max<int64_t>(65536, 64LL * nlist_);
        if (index_param.Contains("train_sample_count")) {
            train_sample_count_ = index_param["train_sample_count"].GetInt();
            CHECK_ARGUMENT(train_sample_count_ >= 512, "train_sample_count must be at least 512");
        }
    }

    Expected<std::vector<int64_t>>
    Build(const DatasetPtr& base) override {
        return safe_call<std::vector<int64_t>>([&]() {
            std::lock_guard<std::mutex> lock(mutex_);
            if (!labels_.empty()) {
                throw VsagException(ErrorType::BUILD_TWICE, "failed to build index: index is not empty");
            }
            return add_locked(base);
        });
    }

    Expected<std::vector<int64_t>>
    Add(const DatasetPtr& base) override {
        return safe_call<std::vector<int64_t>>([&]() {
            std::lock_guard<std::mutex> lock(mutex_);
            return add_locked(base);
        });
    }

protected:
    DatasetPtr
    search(const DatasetPtr& query, int64_t k, const std::string& parameters, const SearchSpec& spec) const override {
        check_query(query, k, q_.dim);
        // IVFSearchParameters::FromJson (src/algorithm/ivf/ivf_parameter.cpp:150-187)
        Json params = Json::Parse(parameters);
        CHECK_ARGUMENT(params.IsObject() && params.Contains("ivf"), "parameters must contains ivf");
        const Json& ivf = params["ivf"];
        CHECK_ARGUMENT(ivf.IsObject() && ivf.Contains("scan_buckets_count"),
                       "parameters[ivf] must contains scan_buckets_count");
        int64_t scan = ivf["scan_buckets_count"].GetInt();
        CHECK_ARGUMENT(scan >= 1, "scan_buckets_count must be positive");
        float factor = 2.0F;
        if (ivf.Contains("factor")) {
            factor = static_cast<float>(ivf["factor"].GetFloat());
        }
        bool enable_reorder = true;
        if (ivf.Contains("enable_reorder")) {
            enable_reorder = ivf["enable_reorder"].GetBool();
        }
        bool disable_scan = ivf.Contains("disable_bucket_scan") && ivf["disable_bucket_scan"].GetBool();

        std::lock_guard<std::mutex> lock(mutex_);
        const int64_t nq = query->GetNumElements();
        if (labels_.empty()) {
            auto empty = Dataset::Make();
            empty->NumElements(1)->Dim(0);
            return empty;
        }
        const auto n = static_cast<int64_t>(labels_.size());
        const auto nprobe = static_cast<uint32_t>(std::min<int64_t>(scan, nlist_));  // ivf.cpp:1573-1574
        const bool reorder = use_reorder_ && enable_reorder;
        if (reorder) {
            CHECK_ARGUMENT(factor > 0.0F, "factor must be positive when use_reorder is true");
        }
        int64_t kcand = k;
        if (reorder && !spec.range) {
            kcand = std::max<int64_t>(static_cast<int64_t>(factor * static_cast<float>(k)), 1);  // ivf.cpp:2316
        }
        // One device scan returns at most 1024 candidates per query; more (and every range search) run scan
        // after scan for one query, each denied what the earlier ones returned.
        const bool looped = spec.range || kcand > kMaxDeviceK;
        CHECK_ARGUMENT(!looped || nq == 1, spec.range ? "range search takes one query"
                                                      : "factor * k above 1024 is supported for one query per call");

        queries_.reserve(static_cast<size_t>(nq) * q_.dim * 4);
        dev(vsag_amd_memcpy_h2d(queries_.p, query->GetFloat32Vectors(), static_cast<size_t>(nq) * q_.dim * 4, nullptr));
        // 1. route (exact nearest centroids)
        buckets_.reserve(static_cast<size_t>(nq) * nprobe * 4);
        bucket_d_.reserve(static_cast<size_t>(nq) * nprobe * 4);
        size_t wsb = vsag_amd_ivf_route_workspace_bytes(centroid_store_.s, nq, nprobe);
        workspace_.reserve(wsb);
        dev(vsag_amd_ivf_route(centroid_store_.s, queries_.as<float>(), nq, nprobe, buckets_.as<int32_t>(),
                               bucket_d_.as<float>(), workspace_.p, wsb, nullptr));
        if (disable_scan && !spec.range) {
            // routing only: bucket ids + centroid distances (ivf.cpp:1589-1660)
            std::vector<uint32_t> ids(static_cast<size_t>(nq) * nprobe);
            std::vector<float> dists(ids.size());
            dev(vsag_amd_memcpy_d2h(ids.data(), buckets_.p, ids.size() * 4, nullptr));
            dev(vsag_amd_memcpy_d2h(dists.data(), bucket_d_.p, dists.size() * 4, nullptr));
            std::vector<int64_t> identity(nlist_);
            for (uint32_t i = 0; i < nlist_; ++i) {
                identity[i] = i;
            }
            return pack_results(ids, dists, nq, nprobe, identity, "{}");
        }
        DenyMask mask;
        mask.init(labels_, spec.valid, looped);
        // FlatBucketSearcher compares against radius + THRESHOLD_ERROR (flat_bucket_searcher.cpp:121,
        // impl/searcher/basic_searcher.h:39).
        const vsag_amd_search_options_t opt = mask.options(spec, 2e-6F);

        if (!looped) {
            // 2. scan the probed lists; 3. exact rerank, best min(k, candidates) kept (flatten_reorder.cpp:77)
            const int64_t kout = reorder ? std::min<int64_t>(k, kcand) : kcand;
            std::vector<uint32_t> ids;
            std::vector<float> dists;
            scan_lists(nq, nprobe, static_cast<uint32_t>(kcand), opt, reorder ? static_cast<uint32_t>(kout) : 0U, ids,
                       dists);
            return pack_results(ids, dists, nq, kout, labels_, "{}");
        }
        // Range (ivf.cpp:2282-2307): candidates within the radius by the list codes, at most factor *
        // limited_size of them when a rerank follows; the rerank keeps the nearest limited_size (all of them
        // when unlimited).  Large k: kcand candidates, the rerank keeps k.
        int64_t want = kcand;
        int64_t keep = k;
        if (spec.range) {
            want = spec.limited_size > 0 ? spec.limited_size : n;
            keep = want;
            if (reorder && spec.limited_size > 0) {
                want = std::max<int64_t>(static_cast<int64_t>(factor * static_cast<float>(spec.limited_size)), 1);
            }
        }
        std::vector<std::pair<float, uint32_t>> row;
        int64_t remaining = want;
        while (remaining > 0) {
            const auto kc = static_cast<uint32_t>(std::min<int64_t>({remaining, kMaxDeviceK, n}));
            std::vector<uint32_t> ids;
            std::vector<float> dists;
            scan_lists(1, nprobe, kc, opt, reorder ? kc : 0U, ids, dists);
            uint32_t got = 0;
            while (got < kc && ids[got] != VSAG_AMD_INVALID_ID) {
                row.emplace_back(dists[got], ids[got]);
                mask.deny(ids[got]);
                ++got;
            }
            remaining -= got;
            if (got < kc) {
                break;
            }
            mask.upload();
        }
        if (reorder) {
            // batches were reranked one by one: order the whole row by exact distance
            std::sort(row.begin(), row.end());
            if (static_cast<int64_t>(row.size()) > keep) {
                row.resize(static_cast<size_t>(keep));
            }
        }
        if (row.empty()) {
            auto empty = Dataset::Make();
            empty->NumElements(1)->Dim(0)->Statistics("{}");
            return empty;
        }
        return pack_row(row, labels_, "{}");
    }

public:
    int64_t
    GetNumElements() const override {
        std::lock_guard<std::mutex> lock(mutex_);
        return static_cast<int64_t>(labels_.size());
    }

private:
    // Scan of the routed lists for the uploaded queries, then (rerank_k > 0) the exact fp32 rerank that keeps
    // rerank_k; results copied to the host, kcand or rerank_k per query.
    void
    scan_lists(int64_t nq, uint32_t nprobe, uint32_t kcand, const vsag_amd_search_options_t& opt, uint32_t rerank_k,
               std::vector<uint32_t>& ids, std::vector<float>& dists) const {
        cand_ids_.reserve(static_cast<size_t>(nq) * kcand * 4);
        cand_d_.reserve(static_cast<size_t>(nq) * kcand * 4);
        size_t wsb = vsag_amd_ivf_scan_workspace_bytes(lists_.s, nq, nprobe, kcand);
        workspace_.reserve(wsb);
        dev(vsag_amd_ivf_scan_topk_ex(lists_.s, queries_.as<float>(), nq, buckets_.as<int32_t>(), nprobe, kcand, &opt,
                                      cand_ids_.as<uint32_t>(), cand_d_.as<float>(), workspace_.p, wsb, nullptr));
        const DevBuf* final_ids = &cand_ids_;
        const DevBuf* final_d = &cand_d_;
        uint32_t kout = kcand;
        if (rerank_k > 0) {
            kout = rerank_k;
            out_ids_.reserve(static_cast<size_t>(nq) * kout * 4);
            out_d_.reserve(static_cast<size_t>(nq) * kout * 4);
            dev(vsag_amd_rerank_fp32(raw_.as<float>(), labels_.size(), q_.dim, q_.metric, queries_.as<float>(), nq,
                                     cand_ids_.as<uint32_t>(), kcand, kout, out_ids_.as<uint32_t>(), out_d_.as<float>(),
                                     nullptr));
            final_ids = &out_ids_;
            final_d = &out_d_;
        }
        ids.resize(static_cast<size_t>(nq) * kout);
        dists.resize(ids.size());
        dev(vsag_amd_memcpy_d2h(ids.data(), final_ids->p, ids.size() * 4, nullptr));
        dev(vsag_amd_memcpy_d2h(dists.data(), final_d->p, dists.size() * 4, nullptr));
    }

    // IVF::Train (ivf.cpp:564-588): sample, k-means (25 iterations, hard-coded in
    // ivf_nearest_partition.cpp:65-70), quantizer training on the same sample.
    void
    train(const DatasetPtr& base, const std::vector<int64_t>& rows, const DevBuf& x_all) {
        const uint64_t n = rows.size();
        uint64_t sample_n = std::min<uint64_t>(n, static_cast<uint64_t>(train_sample_count_));
        if (n < nlist_) {
            throw VsagException(ErrorType::INVALID_ARGUMENT, "k cannot be larger than count");
        }
        // Seeded choice without replacement (the reference reservoir-samples from std::random_device,
        // utils/util_functions.cpp:274-319).
        std::mt19937_64 gen(47);
        std::vector<uint64_t> perm(n);
        for (uint64_t i = 0; i < n; ++i) {
            perm[i] = i;
        }
        for (uint64_t i = 0; i < sample_n; ++i) {
            std::uniform_int_distribution<uint64_t> dis(i, n - 1);
            std::swap(perm[i], perm[dis(gen)]);
        }
        const float* src = base->GetFloat32Vectors();
        std::vector<float> sample(sample_n * q_.dim);
        for (uint64_t i = 0; i < sample_n; ++i) {
            std::memcpy(sample.data() + i * q_.dim, src + rows[perm[i]] * q_.dim, static_cast<size_t>(q_.dim) * 4);
        }
        DevBuf sample_dev;
        sample_dev.reserve(sample.size() * 4);
        dev(vsag_amd_memcpy_h2d(sample_dev.p, sample.data(), sample.size() * 4, nullptr));
        // Initial centroids: the first nlist rows of the shuffled sample (random-sample initialisation;
        // the reference defaults to k-means++ drawn from std::random_device).
        centroids_.reserve(static_cast<size_t>(nlist_) * q_.dim * 4);
        dev(vsag_amd_memcpy_d2d(centroids_.p, sample_dev.p, static_cast<size_t>(nlist_) * q_.dim * 4, nullptr));
        if (!train_random_) {
            DevBuf labels, ws;
            labels.reserve(sample_n * 4);
            size_t wsb = vsag_amd_kmeans_run_workspace_bytes(sample_n, q_.dim, nlist_);
            ws.reserve(wsb);
            double loss = 0;
            dev(vsag_amd_kmeans_run(sample_dev.as<float>(), sample_n, q_.dim, centroids_.as<float>(), nlist_, 25, 47,
                                    labels.as<int32_t>(), &loss, ws.p, wsb, nullptr));
        }
        // Router: an fp32 store of the centroids under the index metric (cosine normalises them,
        // ivf_nearest_partition.cpp:81-85).
        Quantizer cq;
        cq.kind = VSAG_AMD_KIND_FP32;
        cq.metric = q_.metric;
        cq.dim = q_.dim;
        centroid_store_.s = cq.make_store();
        dev(vsag_amd_store_append(centroid_store_.s, centroids_.as<uint8_t>(), nlist_, nullptr));
        q_.train(sample_dev.as<float>(), sample_n);
        lists_.s = q_.make_store();
        dev(vsag_amd_stream_synchronize(nullptr));
        (void)x_all;
        trained_ = true;
    }

    std::vector<int64_t>
    add_locked(const DatasetPtr& base) {
        check_base(base, q_.dim);
        std::vector<int64_t> rows;
        std::vector<int64_t> failed = split_new_rows(base, known_, rows);
        if (rows.empty()) {
            return failed;
        }
        const uint64_t n_new = rows.size();
        const uint64_t n_old = labels_.size();
        DevBuf x;
        upload_rows(base, rows, q_.dim, x);
        if (!trained_) {
            try {
                train(base, rows, x);
            } catch (...) {
                for (int64_t r : rows) {
                    known_.erase(base->GetIds()[r]);
                }
                throw;
            }
        }
        // IVFPartitionStrategy::ClassifyDatas with exact nearest centroids: k-means assignment always
        // measures plain L2 on the raw vectors (ivf_nearest_partition.cpp:63-70).
        bucket_labels_.grow((n_old + n_new) * 4, n_old * 4);
        {
            DevBuf ws;
            size_t wsb = vsag_amd_kmeans_assign_workspace_bytes(n_new, q_.dim, nlist_);
            ws.reserve(wsb);
            dev(vsag_amd_kmeans_assign(x.as<float>(), n_new, q_.dim, centroids_.as<float>(), nlist_,
                                       bucket_labels_.as<int32_t>() + n_old, nullptr, nullptr, ws.p, wsb, nullptr));
            dev(vsag_amd_stream_synchronize(nullptr));
        }
        // Codes of every vector in inner-id order; the posting lists are rebuilt from them.
        const uint64_t cs = q_.code_size();
        codes_.grow((n_old + n_new) * cs, n_old * cs);
        if (q_.kind == VSAG_AMD_KIND_FP32) {
            dev(vsag_amd_memcpy_d2d(codes_.as<uint8_t>() + n_old * cs, x.p, n_new * cs, nullptr));
        } else {
            q_.encode(x.as<float>(), n_new, codes_.as<uint8_t>() + n_old * cs);
        }
        dev(vsag_amd_store_set_lists(lists_.s, codes_.as<uint8_t>(), bucket_labels_.as<int32_t>(), n_old + n_new,
                                     nlist_, nullptr));
        if (use_reorder_) {
            const size_t row_bytes = static_cast<size_t>(q_.dim) * 4;
            raw_.grow((n_old + n_new) * row_bytes, n_old * row_bytes);
            dev(vsag_amd_memcpy_d2d(raw_.as<uint8_t>() + n_old * row_bytes, x.p, n_new * row_bytes, nullptr));
        }
        dev(vsag_amd_stream_synchronize(nullptr));
        for (int64_t r : rows) {
            labels_.push_back(base->GetIds()[r]);
        }
        return failed;
    }

    CommonParam common_;
    Quantizer q_;
    uint32_t nlist_ = 10;
    bool use_reorder_ = false;
    bool train_random_ = false;
    int64_t train_sample_count_ = 65536;
    bool trained_ = false;
    StoreHandle centroid_store_, lists_;
    DevBuf centroids_, codes_, bucket_labels_, raw_;
    std::vector<int64_t> labels_;
    std::unordered_set<int64_t> known_;
    mutable std::mutex mutex_;
    mutable DevBuf queries_, buckets_, bucket_d_, cand_ids_, cand_d_, out_ids_, out_d_, workspace_;
};

}  // namespace

Expected<std::shared_ptr<Index>>
Factory::CreateIndex(const std::string& name, const std::string& parameters) {
    return safe_call<std::shared_ptr<Index>>([&]() -> std::shared_ptr<Index> {
        Json params = Json::Parse(parameters);
        CommonParam common = parse_common(params);
        Json index_param;
        index_param.type = Json::Type::Object;
        if (params.Contains("index_param")) {
            index_param = params["index_param"];
            CHECK_ARGUMENT(index_param.IsObject(), "parameters[index_param] must be a JSON object");
        }
        // The constructors only validate parameters; the device is touched afterwards, so that parameter
        // errors are reported the same way with or without a GPU.
        std::shared_ptr<Index> index;
        if (name == "brute_force") {
            index = std::make_shared<BruteForce>(common, index_param);
        } else if (name == "ivf") {
            index = std::make_shared<IVF>(common, index_param);
        }
        if (index != nullptr) {
            static std::once_flag once;
            static int init_rc = 0;
            static std::string init_message;
            std::call_once(once, []() {
                init_rc = vsag_amd_init(0);
                if (init_rc != 0) {
                    init_message = vsag_amd_last_error();
                }
            });
            if (init_rc != 0) {
                throw VsagException(ErrorType::INTERNAL_ERROR, init_message);
            }
            return index;
        }
        throw VsagException(ErrorType::UNSUPPORTED_INDEX, "failed to create index(unsupported): " + name);
    });
}

}  // namespace vsag
