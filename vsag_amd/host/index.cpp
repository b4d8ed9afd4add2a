// brute_force and ivf index classes on top of the HIP library: the host side of
//   BruteForce  (src/algorithm/bruteforce/bruteforce.cpp:91-95,213-293,354-635,1142-1376)
//   IVF         (src/algorithm/ivf/ivf.cpp:78-410,548-724,892-907,1565-1587,2052-2354)
//   Factory / Engine / IndexImpl error mapping (src/factory/engine.cpp:49-68, src/index/index_impl.h:309-322)
// It owns parameter parsing, the label table, Dataset packing and error mapping; every distance, every
// code and every centroid is computed by libvsag_amd.so.  There is no host arithmetic to fall back to.
#include <algorithm>
#include <cmath>
#include <condition_variable>
#include <cstring>
#include <functional>
#include <istream>
#include <limits>
#include <map>
#include <mutex>
#include <ostream>
#include <shared_mutex>
#include <random>
#include <set>
#include <stdexcept>
#include <unordered_map>
#include <unordered_set>

#include "../../include/vsag_amd.h"
#include "json.h"
#include "vsag_host.h"

namespace vsag {
inline namespace amd_gpu {
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

template <typename F>
Expected<void>
safe_run(F&& f) {
    try {
        f();
        return Expected<void>();
    } catch (const VsagException& e) {
        return Expected<void>(Error(e.type, e.message));
    } catch (const std::bad_alloc&) {
        return Expected<void>(Error(ErrorType::NO_ENOUGH_MEMORY, "not enough memory"));
    } catch (const std::invalid_argument& e) {
        return Expected<void>(Error(ErrorType::INVALID_ARGUMENT, e.what()));
    } catch (const std::exception& e) {
        return Expected<void>(Error(ErrorType::UNKNOWN_ERROR, e.what()));
    }
}

struct DevBuf {
    void* p = nullptr;
    size_t bytes = 0;
    DevBuf() = default;
    DevBuf(const DevBuf&) = delete;
    DevBuf&
    operator=(const DevBuf&) = delete;
    DevBuf(DevBuf&& other) noexcept : p(other.p), bytes(other.bytes) {
        other.p = nullptr;
        other.bytes = 0;
    }
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

// What one search in flight owns on the device: a stream of its own and its buffers.  Searches are const and may run
// concurrently on one index (SUPPORT_SEARCH_CONCURRENT, bruteforce.cpp:1112-1116, ivf.cpp:498; tools/eval drives one
// query per call from an OpenMP loop, tools/eval/case/search_eval_case.cpp:233-248): each takes a context from the
// index's pool and gives it back, so the buffers are reused without being shared.
//
// Host data crosses through a pinned staging area of the context: an upload copies into it and queues the transfer
// without waiting, a download queues the transfer into it and hands the bytes over at finish(), which is the one
// point where a search waits for the device.  (A copy from or to pageable memory waits on its own, and the caller's
// arrays cannot be pinned after the fact.)  Transfers too large for the area go the plain, waiting way.
struct SearchContext {
    void* stream = nullptr;
    DevBuf queries, buckets, bucket_d, cand_ids, cand_d, out_ids, out_d, workspace, deny, scalar;
    SearchContext() {
        dev(vsag_amd_stream_create(&stream));
    }
    SearchContext(const SearchContext&) = delete;
    SearchContext&
    operator=(const SearchContext&) = delete;
    ~SearchContext() {
        if (stream != nullptr) {
            vsag_amd_stream_synchronize(stream);
            vsag_amd_stream_destroy(stream);
        }
        vsag_amd_host_free(stage_);
    }
    void
    upload(DevBuf& buf, const void* src, size_t n) {
        buf.reserve(std::max<size_t>(n, 4));
        void* s = staged(n);
        if (s == nullptr) {
            dev(vsag_amd_memcpy_h2d(buf.p, src, n, stream));
            return;
        }
        std::memcpy(s, src, n);
        dev(vsag_amd_memcpy_h2d_async(buf.p, s, n, stream));
    }
    // The bytes are in `dst` after the next finish().
    void
    download_later(void* dst, const void* src_dev, size_t n) {
        void* s = staged(n);
        if (s == nullptr) {
            dev(vsag_amd_memcpy_d2h(dst, src_dev, n, stream));
            return;
        }
        dev(vsag_amd_memcpy_d2h_async(s, src_dev, n, stream));
        pending_.push_back({dst, s, n});
    }
    void
    download(void* dst, const void* src_dev, size_t n) {
        download_later(dst, src_dev, n);
        finish();
    }
    // Waits for everything queued on the stream and hands over the downloads.
    void
    finish() {
        dev(vsag_amd_stream_synchronize(stream));
        for (const Pending& p : pending_) {
            std::memcpy(p.dst, p.staged, p.bytes);
        }
        pending_.clear();
        stage_used_ = 0;
    }

private:
    struct Pending {
        void* dst;
        const void* staged;
        size_t bytes;
    };
    static constexpr size_t kStageLimit = 8u << 20;  // larger transfers are not staged
    // Room for n bytes in the pinned area (null: too large).  A full area is emptied by finish() first.
    void*
    staged(size_t n) {
        const size_t need = (n + 63) / 64 * 64;
        if (need > kStageLimit) {
            return nullptr;
        }
        if (stage_used_ + need > stage_cap_) {
            finish();
            if (need > stage_cap_) {
                vsag_amd_host_free(stage_);
                stage_ = nullptr;
                stage_cap_ = 0;
                const size_t cap = std::max<size_t>(need, 1u << 16);
                void* p = nullptr;
                dev(vsag_amd_host_malloc(&p, cap));
                stage_ = static_cast<uint8_t*>(p);
                stage_cap_ = cap;
            }
        }
        void* s = stage_ + stage_used_;
        stage_used_ += need;
        return s;
    }
    uint8_t* stage_ = nullptr;
    size_t stage_cap_ = 0, stage_used_ = 0;
    std::vector<Pending> pending_;
};

class ContextPool {
public:
    class Lease {
    public:
        Lease(ContextPool* pool, std::unique_ptr<SearchContext> ctx) : pool_(pool), ctx_(std::move(ctx)) {
        }
        Lease(Lease&&) = default;
        ~Lease() {
            if (ctx_ != nullptr) {
                std::lock_guard<std::mutex> lock(pool_->mutex_);
                pool_->free_.push_back(std::move(ctx_));
            }
        }
        SearchContext*
        operator->() {
            return ctx_.get();
        }
        SearchContext&
        operator*() {
            return *ctx_;
        }

    private:
        ContextPool* pool_;
        std::unique_ptr<SearchContext> ctx_;
    };

    Lease
    acquire() {
        {
            std::lock_guard<std::mutex> lock(mutex_);
            if (!free_.empty()) {
                auto ctx = std::move(free_.back());
                free_.pop_back();
                return Lease(this, std::move(ctx));
            }
        }
        return Lease(this, std::make_unique<SearchContext>());
    }

private:
    std::mutex mutex_;
    std::vector<std::unique_ptr<SearchContext>> free_;
};

// ------------------------------------------------------------------------------------------- serialized form
// StreamWriter / StreamReader of the reference (src/storage/stream_writer.h:28-60, stream_reader.h): objects as their
// bytes, vectors and strings behind a u64 count.
class Writer {
public:
    explicit Writer(std::ostream& os) : os_(os) {
    }
    void
    write(const void* p, size_t n) {
        os_.write(static_cast<const char*>(p), static_cast<std::streamsize>(n));
        if (!os_) {
            throw VsagException(ErrorType::INTERNAL_ERROR, "writing the serialized index failed");
        }
        cursor_ += n;
    }
    template <typename T>
    void
    obj(const T& v) {
        write(&v, sizeof(T));
    }
    template <typename T>
    void
    vec(const std::vector<T>& v) {
        const uint64_t n = v.size();
        obj(n);
        if (n > 0) {
            write(v.data(), n * sizeof(T));
        }
    }
    void
    str(const std::string& v) {
        const uint64_t n = v.size();
        obj(n);
        write(v.data(), n);
    }
    uint64_t
    cursor() const {
        return cursor_;
    }

private:
    std::ostream& os_;
    uint64_t cursor_ = 0;
};

class Reader {
public:
    explicit Reader(std::istream& is) : is_(is) {
        base_ = is_.tellg();
        is_.seekg(0, std::ios::end);
        const std::streampos end = is_.tellg();
        if (base_ < 0 || end < base_) {
            throw VsagException(ErrorType::READ_ERROR, "the stream of a serialized index must be seekable");
        }
        length_ = static_cast<uint64_t>(end - base_);
        is_.seekg(base_);
    }
    void
    read(void* p, uint64_t n) {
        if (n > length_ - cursor_) {
            throw VsagException(ErrorType::INVALID_BINARY, "the serialized index ends early");
        }
        is_.read(static_cast<char*>(p), static_cast<std::streamsize>(n));
        if (static_cast<uint64_t>(is_.gcount()) != n) {
            throw VsagException(ErrorType::READ_ERROR, "reading the serialized index failed");
        }
        cursor_ += n;
    }
    template <typename T>
    void
    obj(T& v) {
        read(&v, sizeof(T));
    }
    template <typename T>
    T
    get() {
        T v;
        obj(v);
        return v;
    }
    template <typename T>
    void
    vec(std::vector<T>& v) {
        const uint64_t n = get<uint64_t>();
        if (n > (length_ - cursor_) / sizeof(T)) {
            throw VsagException(ErrorType::INVALID_BINARY, "a vector of the serialized index is longer than the stream");
        }
        v.resize(n);
        if (n > 0) {
            read(v.data(), n * sizeof(T));
        }
    }
    uint64_t
    cursor() const {
        return cursor_;
    }
    uint64_t
    length() const {
        return length_;
    }
    void
    seek(uint64_t pos) {
        if (pos > length_) {
            throw VsagException(ErrorType::INVALID_BINARY, "the serialized index ends early");
        }
        is_.clear();
        is_.seekg(base_ + static_cast<std::streamoff>(pos));
        cursor_ = pos;
    }
    void
    skip(uint64_t n) {
        if (n > length_ - cursor_) {
            throw VsagException(ErrorType::INVALID_BINARY, "the serialized index ends early");
        }
        seek(cursor_ + n);
    }

private:
    std::istream& is_;
    std::streampos base_;
    uint64_t length_ = 0;
    uint64_t cursor_ = 0;
};

// Footer (src/storage/serialization.cpp:122-222, serialization.h:193-205):
// [magic "vsag0000"][u64 metadata length][metadata JSON][u32 CRC-32 of the JSON][u64 footer length][cigam "0000gasv"].
uint32_t
footer_checksum(const std::string& bytes) {
    uint32_t crc = 0xFFFFFFFFU;
    for (const char byte : bytes) {
        crc ^= static_cast<uint32_t>(static_cast<int32_t>(byte));  // `crc ^= byte` on a char: sign-extended
        for (int j = 0; j < 8; ++j) {
            crc = (crc >> 1) ^ ((crc & 1U) != 0 ? 0xEDB88320U : 0U);
        }
    }
    return crc ^ 0xFFFFFFFFU;
}

void
write_footer(Writer& w, const std::string& metadata) {
    w.write("vsag0000", 8);
    w.str(metadata);
    w.obj(footer_checksum(metadata));
    const uint64_t length = 8 + 8 + metadata.size() + 4 + 8 + 8;
    w.obj(length);
    w.write("0000gasv", 8);
}

// The metadata JSON of the footer at the end of the stream and the footer's length; false when there is none.
bool
read_footer(Reader& r, std::string* metadata, uint64_t* footer_length) {
    constexpr uint64_t kTrailer = 16, kMin = 36;
    if (r.length() < kMin) {
        return false;
    }
    const uint64_t back = r.cursor();
    char trailer[kTrailer];
    r.seek(r.length() - kTrailer);
    r.read(trailer, kTrailer);
    uint64_t length = 0;
    std::memcpy(&length, trailer, 8);
    bool ok = std::memcmp(trailer + 8, "0000gasv", 8) == 0 && length >= kMin && length <= r.length();
    if (ok) {
        std::vector<char> body(length);
        r.seek(r.length() - length);
        r.read(body.data(), length);
        uint64_t mlen = 0;
        std::memcpy(&mlen, body.data() + 8, 8);
        ok = std::memcmp(body.data(), "vsag0000", 8) == 0 && mlen == length - kMin;
        if (ok) {
            metadata->assign(body.data() + 16, mlen);
            uint32_t crc = 0;
            std::memcpy(&crc, body.data() + 16 + mlen, 4);
            ok = crc == footer_checksum(*metadata);
            *footer_length = length;
        }
    }
    r.seek(back);
    return ok;
}

constexpr uint64_t kIoChunkBytes = 64ull << 20;  // codes cross the host 64 MiB at a time

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
        {"rabitq", VSAG_AMD_KIND_RABITQ}, {"pqfs", VSAG_AMD_KIND_PQFS}};
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
    // RaBitQuantizerParameter (rabitq_quantizer_parameter.h:57-64): bits per dimension of the base code and the encoder
    // of multi-bit codes (FastEncodeRaBitQ with this many rounds, else EncodeExtendRaBitQ).
    int rabitq_base_bits = 1;
    bool rabitq_fast_encode = true;
    uint32_t rabitq_fast_rounds = 6;
    uint32_t pq_dim = 1;  // pqfs: subspaces (PQFastScanQuantizerParameter::pq_dim_, default 1)
    // rabitq_use_fht: the rotation is FhtKacRotator's (fht_kac_rotate_transformer.cpp), kept as its sign bits (what
    // the reference serializes) and handed to the device as the dense matrix it stands for.
    bool rabitq_use_fht = false;
    std::vector<uint8_t> fht_flip;
    bool trained = false;
    DevBuf lb, diff, bounds, rotation, centroid, codebooks;

    int
    rabitq_bits() const {
        return VSAG_AMD_RABITQ_BITS(rabitq_query_bits, rabitq_base_bits);
    }
    uint64_t
    code_size() const {
        return vsag_amd_code_size(kind, metric, kind == VSAG_AMD_KIND_PQFS ? pq_dim : dim, rabitq_bits());
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

    std::vector<float>
    fht_matrix() const {
        std::vector<float> rot(static_cast<size_t>(dim) * dim);
        dev(vsag_amd_fht_kac_matrix(fht_flip.data(), dim, rot.data()));
        return rot;
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
                std::vector<float> rot;
                if (rabitq_use_fht) {
                    // FhtKacRotator::Train (fht_kac_rotate_transformer.cpp:50-57): uniform bytes; seeded here, from
                    // std::random_device there
                    std::mt19937 gen(20240229U);
                    std::uniform_int_distribution<int> byte(0, 255);
                    fht_flip.resize(4 * ((static_cast<size_t>(dim) + 7) / 8));
                    for (auto& b : fht_flip) {
                        b = static_cast<uint8_t>(byte(gen));
                    }
                    rot = fht_matrix();
                } else {
                    rot = random_rotation(dim, 20240229U);
                }
                rotation.reserve(rot.size() * 4);
                centroid.reserve(dim * 4);
                dev(vsag_amd_memcpy_h2d(rotation.p, rot.data(), rot.size() * 4, nullptr));
                dev(vsag_amd_rabitq_train(x_dev, n, dim, rotation.as<float>(), centroid.as<float>(), nullptr));
                break;
            }
            case VSAG_AMD_KIND_PQFS: {
                // PQFastScanQuantizer::TrainImpl (pq_fastscan_quantizer.cpp:62-94); the seed is fixed so that a build
                // is reproducible (the reference draws from std::random_device)
                codebooks.reserve(static_cast<size_t>(dim) * 16 * 4);
                size_t wsb = vsag_amd_pq_train_workspace_bytes(n, dim, pq_dim);
                ws.reserve(wsb);
                dev(vsag_amd_pq_train(x_dev, n, dim, pq_dim, metric, 20240301U, codebooks.as<float>(), ws.p, wsb, nullptr));
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
                if (rabitq_base_bits != 1) {
                    dev(vsag_amd_rabitq_encode_multibit(x_dev, n, dim, rotation.as<float>(), centroid.as<float>(), metric,
                                                        rabitq_bits(), rabitq_fast_encode ? 1 : 0, rabitq_fast_rounds,
                                                        codes, nullptr));
                    break;
                }
                dev(vsag_amd_rabitq_encode(x_dev, n, dim, rotation.as<float>(), centroid.as<float>(), metric,
                                           rabitq_query_bits, codes, nullptr));
                break;
            case VSAG_AMD_KIND_PQFS: {
                DevBuf norms;
                if (metric == VSAG_AMD_METRIC_COSINE) {
                    norms.reserve(n * 4);
                }
                dev(vsag_amd_pq_encode(x_dev, n, dim, pq_dim, codebooks.as<float>(), metric, codes, norms.as<float>(),
                                       nullptr));
                dev(vsag_amd_stream_synchronize(nullptr));  // the scratch goes with this scope
                break;
            }
        }
    }

    // The same parameters, untrained; and taking over what another one was loaded with.
    Quantizer
    blank() const {
        Quantizer q;
        q.kind = kind;
        q.metric = metric;
        q.dim = dim;
        q.rabitq_query_bits = rabitq_query_bits;
        q.rabitq_base_bits = rabitq_base_bits;
        q.rabitq_fast_encode = rabitq_fast_encode;
        q.rabitq_fast_rounds = rabitq_fast_rounds;
        q.pq_dim = pq_dim;
        q.rabitq_use_fht = rabitq_use_fht;
        return q;
    }
    void
    take(Quantizer& other) {
        trained = other.trained;
        std::swap(fht_flip, other.fht_flip);
        for (auto pair : {std::make_pair(&lb, &other.lb), std::make_pair(&diff, &other.diff),
                          std::make_pair(&bounds, &other.bounds), std::make_pair(&rotation, &other.rotation),
                          std::make_pair(&centroid, &other.centroid), std::make_pair(&codebooks, &other.codebooks)}) {
            std::swap(pair.first->p, pair.second->p);
            std::swap(pair.first->bytes, pair.second->bytes);
        }
    }

    // Quantizer::Serialize (src/quantization/quantizer.h:161-168) and the SerializeImpl of each kind
    // (scalar_quantizer.cpp:199-204, sq8_uniform_quantizer.cpp:273-281, sq4_uniform_quantizer.cpp:225-234,
    // rabitq_quantizer.cpp:2245-2252 with random_orthogonal_transformer.cpp:193-196; fp32 writes nothing).
    void
    save(Writer& w) const {
        w.obj(static_cast<uint64_t>(dim));
        w.obj(static_cast<int32_t>(metric));  // MetricType: l2 0, ip 1, cosine 2, as here
        w.obj(code_size());
        w.obj(static_cast<uint8_t>(trained ? 1 : 0));
        auto floats = [&](const DevBuf& buf, size_t n) {
            std::vector<float> v(n, 0.0F);
            if (trained && buf.p != nullptr) {
                dev(vsag_amd_memcpy_d2h(v.data(), buf.p, n * 4, nullptr));
            }
            return v;
        };
        auto up = [](uint64_t v, uint64_t a) { return (v + a - 1) / a * a; };
        switch (kind) {
            case VSAG_AMD_KIND_FP32:
                break;
            case VSAG_AMD_KIND_SQ8:
            case VSAG_AMD_KIND_SQ4:
                w.vec(floats(diff, dim));
                w.vec(floats(lb, dim));
                break;
            case VSAG_AMD_KIND_SQ8_UNIFORM: {
                const std::vector<float> b = floats(bounds, 2);  // lower bound, diff
                const bool norm = metric == VSAG_AMD_METRIC_L2;
                const uint64_t behind = up(dim, norm ? 8 : 4);
                w.obj(b[1]);
                w.obj(b[0]);
                w.obj(static_cast<uint64_t>(0));               // offset_code_
                w.obj(static_cast<uint64_t>(norm ? behind : 0));  // offset_norm_
                w.obj(static_cast<uint64_t>(norm ? 0 : behind));  // offset_sum_
                break;
            }
            case VSAG_AMD_KIND_SQ4_UNIFORM: {
                const std::vector<float> b = floats(bounds, 2);
                const bool norm = metric != VSAG_AMD_METRIC_IP, sum = metric != VSAG_AMD_METRIC_L2;
                const uint64_t align = norm ? 8 : 4;
                uint64_t cur = up((static_cast<uint64_t>(dim) + 1) / 2, align);
                uint64_t off_norm = 0, off_sum = 0, off_codes_sum = 0;
                if (norm) {
                    off_norm = cur;
                    cur += up(8, align);
                }
                if (sum) {
                    off_sum = cur;
                    cur += up(4, align);
                    off_codes_sum = cur;
                }
                w.obj(b[1]);
                w.obj(b[0]);
                w.obj(static_cast<uint64_t>(0));
                w.obj(off_norm);
                w.obj(off_sum);
                w.obj(off_codes_sum);
                break;
            }
            case VSAG_AMD_KIND_RABITQ:
                w.vec(floats(centroid, dim));
                if (rabitq_use_fht) {
                    // FhtKacRotator::Serialize (fht_kac_rotate_transformer.cpp:122-125): the sign bits
                    std::vector<uint8_t> flip = fht_flip;
                    flip.resize(4 * ((static_cast<size_t>(dim) + 7) / 8), 0);
                    w.vec(flip);
                } else {
                    w.vec(floats(rotation, static_cast<size_t>(dim) * dim));
                }
                break;
            case VSAG_AMD_KIND_PQFS:
                // PQFastScanQuantizer::SerializeImpl (pq_fastscan_quantizer.cpp:201-207)
                w.obj(static_cast<int64_t>(pq_dim));
                w.obj(static_cast<int64_t>(dim / pq_dim));
                w.vec(floats(codebooks, static_cast<size_t>(dim) * 16));
                break;
        }
    }

    void
    load(Reader& r) {
        const auto fdim = r.get<uint64_t>();
        const auto fmetric = r.get<int32_t>();
        const auto fsize = r.get<uint64_t>();
        const auto ftrained = r.get<uint8_t>();
        if (fdim != dim || fmetric != metric || fsize != code_size()) {
            throw VsagException(ErrorType::INVALID_ARGUMENT,
                                "the serialized quantizer (dim " + std::to_string(fdim) + ", metric " +
                                    std::to_string(fmetric) + ", code size " + std::to_string(fsize) +
                                    ") does not match the index (dim " + std::to_string(dim) + ", metric " +
                                    std::to_string(metric) + ", code size " + std::to_string(code_size()) + ")");
        }
        auto upload = [&](DevBuf& buf, const std::vector<float>& v, size_t want) {
            if (v.size() != want) {
                throw VsagException(ErrorType::INVALID_BINARY, "a table of the serialized quantizer has the wrong length");
            }
            buf.reserve(std::max<size_t>(want * 4, 4));
            dev(vsag_amd_memcpy_h2d(buf.p, v.data(), want * 4, nullptr));
        };
        std::vector<float> a, b;
        switch (kind) {
            case VSAG_AMD_KIND_FP32:
                break;
            case VSAG_AMD_KIND_SQ8:
            case VSAG_AMD_KIND_SQ4:
                r.vec(a);
                r.vec(b);
                upload(diff, a, dim);
                upload(lb, b, dim);
                break;
            case VSAG_AMD_KIND_SQ8_UNIFORM:
            case VSAG_AMD_KIND_SQ4_UNIFORM: {
                const auto fdiff = r.get<float>();
                const auto flb = r.get<float>();
                r.skip(kind == VSAG_AMD_KIND_SQ4_UNIFORM ? 32 : 24);  // the offsets of the code's fields
                upload(bounds, {flb, fdiff}, 2);
                break;
            }
            case VSAG_AMD_KIND_RABITQ:
                r.vec(a);
                upload(centroid, a, dim);
                if (rabitq_use_fht) {
                    r.vec(fht_flip);
                    if (fht_flip.size() != 4 * ((static_cast<size_t>(dim) + 7) / 8)) {
                        throw VsagException(ErrorType::INVALID_ARGUMENT, "the serialized rotator has " +
                                                                             std::to_string(fht_flip.size()) +
                                                                             " sign bytes, this dimension takes " +
                                                                             std::to_string(4 * ((dim + 7) / 8)));
                    }
                    b = fht_matrix();
                } else {
                    r.vec(b);
                }
                upload(rotation, b, static_cast<size_t>(dim) * dim);
                break;
            case VSAG_AMD_KIND_PQFS: {
                const auto fpq = r.get<int64_t>();
                const auto fsd = r.get<int64_t>();
                if (fpq != static_cast<int64_t>(pq_dim) || fsd != static_cast<int64_t>(dim / pq_dim)) {
                    throw VsagException(ErrorType::INVALID_ARGUMENT,
                                        "the serialized pqfs quantizer has pq_dim " + std::to_string(fpq) +
                                            ", the index " + std::to_string(pq_dim));
                }
                r.vec(a);
                upload(codebooks, a, static_cast<size_t>(dim) * 16);
                break;
            }
        }
        trained = ftrained != 0;
    }

    vsag_amd_store_t*
    make_store() const {
        vsag_amd_store_params_t p{};
        p.kind = kind;
        p.metric = metric;
        p.dim = dim;
        p.rabitq_query_bits = rabitq_bits();
        if (kind == VSAG_AMD_KIND_SQ8 || kind == VSAG_AMD_KIND_SQ4) {
            p.lower_bound_dev = lb.as<float>();
            p.diff_dev = diff.as<float>();
        } else if (kind == VSAG_AMD_KIND_SQ4_UNIFORM || kind == VSAG_AMD_KIND_SQ8_UNIFORM) {
            p.lower_bound_dev = bounds.as<float>();
        } else if (kind == VSAG_AMD_KIND_RABITQ) {
            p.rotation_dev = rotation.as<float>();
            p.centroid_dev = centroid.as<float>();
        } else if (kind == VSAG_AMD_KIND_PQFS) {
            p.pq_dim = pq_dim;
            p.codebooks_dev = codebooks.as<float>();
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

using LabelMap = std::unordered_map<int64_t, uint32_t>;  // label -> inner id (LabelTable)

// Rows of `base` whose ids are new; the ids already present (or repeated inside `base`) are reported back and
// skipped, as BruteForce::Add / IVF::Add do through the label table.  Nothing is recorded yet: the caller adds the
// new labels to the table once the device holds the vectors, so that a failed insert leaves the index as it was.
std::vector<int64_t>
split_new_rows(const DatasetPtr& base, const LabelMap& known, std::vector<int64_t>& rows) {
    std::vector<int64_t> failed;
    std::unordered_set<int64_t> batch;
    const int64_t* ids = base->GetIds();
    for (int64_t i = 0; i < base->GetNumElements(); ++i) {
        if (known.count(ids[i]) == 0 && batch.insert(ids[i]).second) {
            rows.push_back(i);
        } else {
            failed.push_back(ids[i]);
        }
    }
    return failed;
}

// Uploads the selected rows (all rows when nothing was skipped) as one n x dim device matrix, every row `repeat`
// times in a row.
void
upload_rows(const DatasetPtr& base, const std::vector<int64_t>& rows, uint32_t dim, DevBuf& out, uint32_t repeat = 1) {
    const float* src = base->GetFloat32Vectors();
    size_t row_bytes = static_cast<size_t>(dim) * 4;
    out.reserve(std::max<size_t>(rows.size() * row_bytes * repeat, 4));
    if (repeat == 1 && static_cast<int64_t>(rows.size()) == base->GetNumElements()) {
        dev(vsag_amd_memcpy_h2d(out.p, src, rows.size() * row_bytes, nullptr));
        return;
    }
    std::vector<float> staged(rows.size() * dim * repeat);
    for (size_t i = 0; i < rows.size(); ++i) {
        for (uint32_t r = 0; r < repeat; ++r) {
            std::memcpy(staged.data() + (i * repeat + r) * dim, src + rows[i] * dim, row_bytes);
        }
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

// What a search asks for beyond (query, k): a pre-filter on labels, a radius, the buckets to scan.
struct SearchSpec {
    bool range = false;
    float radius = 0.0F;
    int64_t limited_size = -1;
    std::function<bool(int64_t)> valid;  // empty = every label is kept
    const std::vector<std::vector<int64_t>>* bucket_ids = nullptr;
};

// Deny mask over the ids the device scans see (inner ids; posting ids = inner id * per_id + j for an ivf index with
// buckets_per_data = per_id), bit set = filtered out; kept on the host as well so that a range search can add the ids
// it has already returned.
struct DenyMask {
    std::vector<uint32_t> words;
    bool active = false;
    uint32_t per_id = 1;

    void
    init(SearchContext& ctx, const std::vector<int64_t>& labels, const std::function<bool(int64_t)>& valid, bool force,
         uint32_t postings_per_id) {
        active = static_cast<bool>(valid) || force;
        per_id = postings_per_id;
        if (!active) {
            return;
        }
        const size_t bits = labels.size() * per_id;
        words.assign((bits + 31) / 32, 0U);
        if (valid) {
            for (size_t i = 0; i < labels.size(); ++i) {
                if (!valid(labels[i])) {
                    deny(static_cast<uint32_t>(i));
                }
            }
        }
        upload(ctx);
    }
    void
    deny(uint32_t inner_id) {
        for (uint32_t j = 0; j < per_id; ++j) {
            const uint64_t bit = static_cast<uint64_t>(inner_id) * per_id + j;
            words[bit >> 5] |= 1U << (bit & 31);
        }
    }
    void
    upload(SearchContext& ctx) {
        ctx.upload(ctx.deny, words.data(), words.size() * 4);
    }
    vsag_amd_search_options_t
    options(const SearchContext& ctx, const SearchSpec& spec, float radius_slack) const {
        vsag_amd_search_options_t o{};
        o.deny_bits_dev = active ? ctx.deny.as<uint32_t>() : nullptr;
        o.use_radius = spec.range ? 1 : 0;
        o.radius = spec.radius + radius_slack;
        return o;
    }
};

constexpr int64_t kMaxDeviceK = 1024;  // largest k of one device scan

const char*
kind_name(int kind) {
    static const char* names[] = {"fp32", "sq8", "sq4", "sq4_uniform", "sq8_uniform", "rabitq", "pqfs"};
    return kind >= 0 && kind <= VSAG_AMD_KIND_PQFS ? names[kind] : "unknown";
}

// ---- index_param of the footer's basic_info ----
// The creating parameters in the reference's internal form, as Parameter::ToString() dumps them (ivf.cpp:1045,
// bruteforce.cpp:703): a reader rebuilds the parameter object from the string and refuses a file whose parameters its
// own index is not compatible with (ivf.cpp:1201-1208, bruteforce.cpp:887-891).  Written here: the fields those
// CheckCompatibility functions compare, under the reference's keys (inner_string_params.h).

// QuantizerParameter::ToJson of each kind (fp32_quantizer_parameter.cpp:33-37, scalar_quantizer_parameter.h:54-58,
// sq4_uniform_quantizer_parameter.cpp:47-52, sq8_uniform_quantizer_parameter.cpp:30-34,
// rabitq_quantizer_parameter.cpp:116-129, pq_fastscan_quantizer_parameter.cpp:36-41).
std::string
quantization_params_json(const Quantizer& q) {
    std::string s = std::string("{\"type\":\"") + kind_name(q.kind) + "\"";
    if (q.kind == VSAG_AMD_KIND_SQ4_UNIFORM) {
        s += ",\"sq4_uniform_trunc_rate\":0.05";
    } else if (q.kind == VSAG_AMD_KIND_PQFS) {
        s += ",\"pq_dim\":" + std::to_string(q.pq_dim);
    } else if (q.kind == VSAG_AMD_KIND_RABITQ) {
        s += ",\"pca_dim\":0,\"rabitq_version\":\"standard\",\"rabitq_bits_per_dim_query\":" +
             std::to_string(q.rabitq_query_bits) + ",\"rabitq_bits_per_dim_base\":" + std::to_string(q.rabitq_base_bits) +
             ",\"rabitq_bits_per_dim_filter\":1,\"rabitq_error_rate\":1.9,\"use_fht\":" +
             (q.rabitq_use_fht ? "true" : "false") + ",\"fast_encode_rabitq\":" +
             (q.rabitq_fast_encode ? "true" : "false") +
             ",\"fast_encode_rabitq_rounds\":" + std::to_string(q.rabitq_fast_rounds);
    }
    return s + "}";
}

// FlattenDataCellParameter::ToJson (flatten_datacell_parameter.cpp:87-97).
std::string
flatten_params_json(const Quantizer& q) {
    return "{\"codes_type\":\"flatten\",\"io_params\":{\"type\":\"block_memory_io\"},\"quantization_params\":" +
           quantization_params_json(q) + "}";
}

// A JSON text as the value of a JSON string.
std::string
json_quoted(const std::string& text) {
    std::string s = "\"";
    for (char c : text) {
        if (c == '"' || c == '\\') {
            s += '\\';
        }
        s += c;
    }
    return s + "\"";
}

// The CheckCompatibility of the quantizer parameters: the same type, and the fields each kind compares
// (sq4_uniform_quantizer_parameter.cpp:54-58, rabitq_quantizer_parameter.cpp:131-141,
// pq_fastscan_quantizer_parameter.cpp:43-48).  Fields a file does not carry are not compared.
bool
quantization_params_compatible(const Json& file, const Quantizer& q) {
    if (!file.IsObject() || !file.Contains("type") || file["type"].GetString() != kind_name(q.kind)) {
        return false;
    }
    auto same_int = [&](const char* key, int64_t mine) { return !file.Contains(key) || file[key].GetInt() == mine; };
    if (q.kind == VSAG_AMD_KIND_SQ4_UNIFORM && file.Contains("sq4_uniform_trunc_rate") &&
        std::fabs(file["sq4_uniform_trunc_rate"].GetFloat() - 0.05) > 1e-6) {
        return false;
    }
    if (q.kind == VSAG_AMD_KIND_PQFS && !same_int("pq_dim", q.pq_dim)) {
        return false;
    }
    if (q.kind == VSAG_AMD_KIND_RABITQ) {
        if (!same_int("rabitq_bits_per_dim_query", q.rabitq_query_bits) ||
            !same_int("rabitq_bits_per_dim_base", q.rabitq_base_bits) || !same_int("rabitq_bits_per_dim_filter", 1)) {
            return false;
        }
        if (file.Contains("pca_dim") && file["pca_dim"].GetInt() != 0 && file["pca_dim"].GetInt() != q.dim) {
            return false;
        }
        if (file.Contains("rabitq_version") && file["rabitq_version"].GetString() != "standard") {
            return false;
        }
        if (file.Contains("use_fht") && file["use_fht"].GetBool() != q.rabitq_use_fht) {
            return false;
        }
    }
    return true;
}

// InnerIndexParameter::CheckCompatibility (inner_index_parameter.cpp:275-286) for an index without attribute filters
// whose reorder source is its precise codes.
bool
inner_params_compatible(const Json& file, bool use_reorder, const Quantizer& precise) {
    if (file.Contains("use_reorder") && file["use_reorder"].GetBool() != use_reorder) {
        return false;
    }
    if (file.Contains("reorder_source") && file["reorder_source"].GetString() != "precise") {
        return false;
    }
    if (use_reorder && file.Contains("precise_codes")) {
        const Json& pc = file["precise_codes"];
        if (pc.Contains("codes_type") && pc["codes_type"].GetString() != "flatten" &&
            pc["codes_type"].GetString() != "flatten_codes") {
            return false;
        }
        if (pc.Contains("quantization_params") && !quantization_params_compatible(pc["quantization_params"], precise)) {
            return false;
        }
    }
    if (file.Contains("use_attribute_filter") && file["use_attribute_filter"].GetBool()) {
        return false;
    }
    if (file.Contains("label_remap_type") && file["label_remap_type"].GetString() != "pg") {
        return false;
    }
    return true;
}

// SearchStatistics::ToJson (src/query_context.h:215-246): distance evaluations of one call by phase and backend.  The
// device scans do not count comparisons one by one; the figures are what the call's plan evaluates: every centroid per
// query (routing), every code of the scanned lists or of the store (approximate), every candidate handed to the
// rerank (at most; a list shorter than the candidate count hands over less).
struct SearchStats {
    uint64_t routing = 0, approximate = 0, rerank = 0;
    int base_kind = VSAG_AMD_KIND_FP32, precise_kind = VSAG_AMD_KIND_FP32;

    std::string
    dump() const {
        std::map<std::string, uint64_t> backend;
        backend["fp32"] += routing;
        backend[kind_name(base_kind)] += approximate;
        backend[kind_name(precise_kind)] += rerank;
        const uint64_t total = routing + approximate + rerank;
        std::string s = "{\"is_timeout\":false,\"dist_cmp\":" + std::to_string(std::min<uint64_t>(total, 0xFFFFFFFFULL)) +
                        ",\"hops\":0,\"io_cnt\":0,\"io_time_ms\":0,\"reorder_distance_count\":" +
                        std::to_string(std::min<uint64_t>(rerank, 0xFFFFFFFFULL)) +
                        ",\"distance_evaluations\":" + std::to_string(total) +
                        ",\"distance_evaluations_by_phase\":{\"routing\":" + std::to_string(routing) +
                        ",\"approximate\":" + std::to_string(approximate) + ",\"rerank\":" + std::to_string(rerank) +
                        "},\"distance_evaluations_by_backend\":{";
        bool first = true;
        for (const auto& b : backend) {
            if (b.second == 0) {
                continue;
            }
            s += std::string(first ? "" : ",") + "\"" + b.first + "\":" + std::to_string(b.second);
            first = false;
        }
        s += "},\"complete\":true}";
        return s;
    }
};

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

// ApplyTopkWithValidity (src/algorithm/inner_index_interface.cpp:611-669): the distances of CalDistanceById as they
// are (topk == -1) or the topk smallest per row with their labels; unknown labels (distance -1) come last, NaN
// distances before them.  inner[i] == VSAG_AMD_INVALID_ID marks an unknown label.
DatasetPtr
pack_distances(const std::vector<float>& dists, const std::vector<uint32_t>& inner, const int64_t* ids, int64_t rows,
               int64_t count, int64_t topk) {
    auto result = Dataset::Make();
    const int64_t out_count = topk == -1 ? count : std::min(topk, count);
    result->NumElements(rows)->Dim(out_count)->Owner(true);
    if (count == 0) {
        return result;
    }
    auto* out_d = new float[rows * out_count];
    result->Distances(out_d);
    if (topk == -1) {
        std::copy(dists.begin(), dists.begin() + rows * count, out_d);
        return result;
    }
    auto* out_ids = new int64_t[rows * out_count];
    result->Ids(out_ids);
    std::vector<int64_t> order(count);
    for (int64_t r = 0; r < rows; ++r) {
        const float* d = dists.data() + r * count;
        const uint32_t* in = inner.data() + r * count;
        for (int64_t i = 0; i < count; ++i) {
            order[i] = i;
        }
        std::partial_sort(order.begin(), order.begin() + out_count, order.end(), [&](int64_t a, int64_t b) {
            const bool va = in[a] != VSAG_AMD_INVALID_ID, vb = in[b] != VSAG_AMD_INVALID_ID;
            if (va != vb) {
                return va;
            }
            const bool na = std::isnan(d[a]), nb = std::isnan(d[b]);
            if (na != nb) {
                return !na;
            }
            if (na) {
                return a < b;
            }
            return d[a] < d[b];
        });
        for (int64_t i = 0; i < out_count; ++i) {
            out_d[r * out_count + i] = d[order[i]];
            out_ids[r * out_count + i] = ids[r * count + order[i]];
        }
    }
    return result;
}

// The search overloads of the public interface, reduced to one virtual search().
// The arrays of a result moved into the caller's allocator (an index created with one hands out only such results).
DatasetPtr
rehome(const DatasetPtr& result, Allocator* allocator) {
    if (allocator == nullptr || result == nullptr) {
        return result;
    }
    const int64_t cells = result->GetNumElements() * result->GetDim();
    auto moved = Dataset::Make();
    moved->NumElements(result->GetNumElements())->Dim(result->GetDim())->Statistics(result->GetStatistics());
    moved->Owner(true, allocator);
    auto copy = [&](const auto* src) -> decltype(src) {
        using T = std::remove_const_t<std::remove_pointer_t<decltype(src)>>;
        if (src == nullptr) {
            return nullptr;
        }
        auto* dst = static_cast<T*>(allocator->Allocate(sizeof(T) * static_cast<uint64_t>(std::max<int64_t>(cells, 1))));
        if (dst == nullptr) {
            throw VsagException(ErrorType::NO_ENOUGH_MEMORY, "the allocator returned no memory for a search result");
        }
        std::copy(src, src + cells, dst);
        return dst;
    };
    moved->Ids(copy(result->GetIds()));
    moved->Distances(copy(result->GetDistances()));
    return moved;
}

class GpuIndex : public Index {
public:
    void
    set_allocator(Allocator* allocator) {
        allocator_ = allocator;
    }
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

    // BruteForce::SearchWithRequest / IVF::SearchWithRequest (bruteforce.cpp:481-597, ivf.cpp:2052-2354): mode, k or
    // radius, parameters, the bitset and the filter object (both, when both are enabled), injected buckets.
    Expected<DatasetPtr>
    SearchWithRequest(const SearchRequest& request) const override {
        SearchSpec spec = request.mode_ == SearchMode::RANGE_SEARCH ? range_spec(request.radius_, request.limited_size_)
                                                                   : SearchSpec{};
        const BitsetPtr bits = request.enable_bitset_filter_ ? request.bitset_filter_ : nullptr;
        const FilterPtr filter = request.enable_filter_ ? request.filter_ : nullptr;
        if (bits != nullptr || filter != nullptr) {
            spec.valid = [bits, filter](int64_t label) {
                return (bits == nullptr || !bits->Test(label & 0xFFFFFFFFLL)) &&
                       (filter == nullptr || filter->CheckValid(label));
            };
        }
        if (!request.bucket_ids_.empty()) {
            spec.bucket_ids = &request.bucket_ids_;
        }
        return run(request.query_, spec.range ? 1 : request.topk_, request.params_str_, spec);
    }

    Expected<DatasetPtr>
    CalDistanceById(const float* query, const int64_t* ids, int64_t count, bool calculate_precise_distance,
                    int64_t topk) const override {
        return safe_call<DatasetPtr>([&]() {
            CHECK_ARGUMENT(count >= 0, "CalDistanceById count must be non-negative");
            CHECK_ARGUMENT(topk == -1 || topk > 0, "CalDistanceById topk must be -1 or positive");
            if (count > 0) {
                CHECK_ARGUMENT(query != nullptr, "CalDistanceById query must not be null");
                CHECK_ARGUMENT(ids != nullptr, "CalDistanceById ids must not be null");
            }
            return rehome(distances_by_id(query, 1, ids, count, calculate_precise_distance, topk), allocator_);
        });
    }
    Expected<DatasetPtr>
    CalDistanceById(const DatasetPtr& query, const int64_t* ids, int64_t count, bool calculate_precise_distance,
                    int64_t topk) const override {
        return safe_call<DatasetPtr>([&]() {
            CHECK_ARGUMENT(query != nullptr, "CalDistanceById query must not be null");
            CHECK_ARGUMENT(count >= 0, "CalDistanceById count must be non-negative");
            CHECK_ARGUMENT(topk == -1 || topk > 0, "CalDistanceById topk must be -1 or positive");
            CHECK_ARGUMENT(query->GetNumElements() > 0, "CalDistanceById query count must be positive");
            if (count > 0) {
                CHECK_ARGUMENT(ids != nullptr, "CalDistanceById ids must not be null");
                CHECK_ARGUMENT(query->GetFloat32Vectors() != nullptr, "query.float_vector is nullptr");
                CHECK_ARGUMENT(query->GetDim() == static_cast<int64_t>(dimension()), "query.dim must be equal to index.dim");
            }
            return rehome(distances_by_id(query->GetFloat32Vectors(), query->GetNumElements(), ids, count,
                                          calculate_precise_distance, topk),
                          allocator_);
        });
    }

    // Index::Serialize(std::ostream&) / Deserialize(std::istream&) (include/vsag/index.h:903-940); the stream of a
    // Deserialize must be seekable (the footer is at its end), the index empty.
    Expected<void>
    Serialize(std::ostream& out) const override {
        return safe_run([&]() {
            std::shared_lock<std::shared_mutex> lock(mutex_);
            Writer w(out);
            save(w);
        });
    }
    Expected<void>
    Deserialize(std::istream& in) override {
        return safe_run([&]() {
            std::unique_lock<std::shared_mutex> lock(mutex_);
            Reader r(in);
            load(r);
        });
    }

protected:
    virtual void
    save(Writer& w) const = 0;
    virtual void
    load(Reader& r) = 0;
    virtual DatasetPtr
    search(const DatasetPtr& query, int64_t k, const std::string& parameters, const SearchSpec& spec) const = 0;
    // rows x count distances (row r: query r against ids[r * count ...]), packed by pack_distances.
    virtual DatasetPtr
    distances_by_id(const float* queries, int64_t rows, const int64_t* ids, int64_t count, bool precise,
                    int64_t topk) const = 0;
    virtual uint32_t
    dimension() const = 0;

    // Searches share the lock; Build / Add / Train hold it alone (bruteforce.cpp:373,1386).
    mutable std::shared_mutex mutex_;
    mutable ContextPool pool_;
    Allocator* allocator_ = nullptr;

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
            if (combinable(query, k, spec)) {
                return rehome(search_combined(query, k, parameters), allocator_);
            }
            return rehome(search(query, k, parameters, spec), allocator_);
        });
    }

    // ---- single queries of concurrent callers, combined ---------------------------------------------------------
    // The reference's evaluator and its users call KnnSearch with one query from many threads
    // (tools/eval/case/search_eval_case.cpp:233-248).  A device scan of one query leaves most of the machine idle and
    // a scan of sixteen costs little more, so plain single-query calls that meet here are served together: a caller
    // that finds no search under way becomes the leader, takes every queued call with its own k and parameters,
    // runs them as one batch (whose rows equal the single-query results bit for bit) and hands the rows out; calls
    // that arrive meanwhile queue up for the next leader.  Up to kCombineLeaders batches are under way at a time (each
    // on a stream of its own), so the device works on one while the host prepares and unpacks others.  A lone caller
    // pays two uncontended lock operations.
    // The statistics of a combined call are the batch's, divided evenly among its queries.
    struct PendingCall {
        const float* query;
        int64_t k;
        const std::string* parameters;
        DatasetPtr result;
        std::exception_ptr error;
        bool taken = false;  // in some leader's batch
        bool done = false;
    };
    mutable std::mutex combine_mutex_;
    mutable std::condition_variable combine_cv_;
    mutable std::vector<PendingCall*> combine_queue_;
    mutable int combine_leaders_ = 0;
    static constexpr int kCombineLeaders = 3;
    static constexpr size_t kCombineMax = 64;

    bool
    combinable(const DatasetPtr& query, int64_t k, const SearchSpec& spec) const {
        return !spec.range && !spec.valid && spec.bucket_ids == nullptr && query != nullptr &&
               query->GetNumElements() == 1 && query->GetFloat32Vectors() != nullptr &&
               query->GetDim() == static_cast<int64_t>(dimension()) && k >= 1 && k <= kMaxDeviceK;
    }

    // Every integer of a statistics string divided by `parts` (they are all counts of one batch).
    static std::string
    divide_counts(const std::string& stats, uint64_t parts) {
        std::string out;
        bool quoted = false;
        for (size_t i = 0; i < stats.size();) {
            const char c = stats[i];
            if (c == '"') {
                quoted = !quoted;
            }
            if (!quoted && c >= '0' && c <= '9') {
                uint64_t v = 0;
                while (i < stats.size() && stats[i] >= '0' && stats[i] <= '9') {
                    v = v * 10 + static_cast<uint64_t>(stats[i] - '0');
                    ++i;
                }
                out += std::to_string(v / parts);
                continue;
            }
            out += c;
            ++i;
        }
        return out;
    }

protected:
    // A batch whose k (or candidate count) is beyond one device scan: the queries one at a time, each through the
    // scan-after-scan loop a single query takes, assembled into the batch form (k columns, -1 / inf behind a row's end).
    DatasetPtr
    search_rows_one_by_one(const DatasetPtr& query, int64_t k, const std::string& parameters, const SearchSpec& spec) const {
        const int64_t nq = query->GetNumElements();
        const int64_t dim = query->GetDim();
        const size_t cells = static_cast<size_t>(nq) * static_cast<size_t>(k);
        std::unique_ptr<int64_t[]> ids(new int64_t[cells]);
        std::unique_ptr<float[]> dists(new float[cells]);
        std::fill(ids.get(), ids.get() + cells, static_cast<int64_t>(-1));
        std::fill(dists.get(), dists.get() + cells, std::numeric_limits<float>::infinity());
        std::string stats;
        for (int64_t i = 0; i < nq; ++i) {
            auto one = Dataset::Make();
            one->Owner(false)->Dim(dim)->NumElements(1)->Float32Vectors(query->GetFloat32Vectors() + i * dim);
            SearchSpec own = spec;
            std::vector<std::vector<int64_t>> own_buckets(1);
            if (spec.bucket_ids != nullptr && static_cast<size_t>(i) < spec.bucket_ids->size()) {
                own_buckets[0] = (*spec.bucket_ids)[static_cast<size_t>(i)];
                own.bucket_ids = &own_buckets;
            }
            const DatasetPtr found = search(one, k, parameters, own);
            const int64_t count = std::min<int64_t>(found->GetDim(), k);
            if (found->GetNumElements() == 1 && count > 0) {
                std::copy(found->GetIds(), found->GetIds() + count, ids.get() + i * k);
                std::copy(found->GetDistances(), found->GetDistances() + count, dists.get() + i * k);
            }
            if (i == 0) {
                stats = found->GetStatistics();
            }
        }
        auto result = Dataset::Make();
        result->NumElements(nq)->Dim(k)->Ids(ids.release())->Distances(dists.release())->Owner(true)->Statistics(stats);
        return result;
    }

private:
    DatasetPtr
    search_combined(const DatasetPtr& query, int64_t k, const std::string& parameters) const {
        PendingCall mine{query->GetFloat32Vectors(), k, &parameters, nullptr, nullptr, false, false};
        std::vector<PendingCall*> batch;
        {
            std::unique_lock<std::mutex> lock(combine_mutex_);
            combine_queue_.push_back(&mine);
            combine_cv_.wait(lock,
                             [&]() { return mine.done || (!mine.taken && combine_leaders_ < kCombineLeaders); });
            if (mine.done) {
                if (mine.error) {
                    std::rethrow_exception(mine.error);
                }
                return mine.result;
            }
            ++combine_leaders_;
            // this call and every queued one with the same k and parameters
            std::vector<PendingCall*> rest;
            batch.push_back(&mine);
            mine.taken = true;
            for (PendingCall* c : combine_queue_) {
                if (c == &mine) {
                    continue;
                }
                if (batch.size() < kCombineMax && c->k == k && *c->parameters == parameters) {
                    c->taken = true;
                    batch.push_back(c);
                } else {
                    rest.push_back(c);
                }
            }
            combine_queue_.swap(rest);
        }
        auto release = [&]() {
            std::lock_guard<std::mutex> lock(combine_mutex_);
            for (PendingCall* c : batch) {
                c->done = true;
            }
            --combine_leaders_;
            combine_cv_.notify_all();
        };
        try {
            if (batch.size() == 1) {
                mine.result = search(query, k, parameters, SearchSpec{});
            } else {
                const uint32_t dim = dimension();
                std::vector<float> rows(batch.size() * dim);
                for (size_t i = 0; i < batch.size(); ++i) {
                    std::memcpy(rows.data() + i * dim, batch[i]->query, static_cast<size_t>(dim) * 4);
                }
                auto all = Dataset::Make();
                all->Owner(false)->Dim(dim)->NumElements(static_cast<int64_t>(batch.size()))->Float32Vectors(rows.data());
                const DatasetPtr found = search(all, k, parameters, SearchSpec{});
                const std::string stats = divide_counts(found->GetStatistics(), batch.size());
                const int64_t cols = found->GetDim();
                const bool none = found->GetNumElements() < static_cast<int64_t>(batch.size());  // an empty index
                for (size_t i = 0; i < batch.size(); ++i) {
                    int64_t count = 0;
                    if (!none) {
                        const int64_t* ids = found->GetIds() + static_cast<int64_t>(i) * cols;
                        const float* ds = found->GetDistances() + static_cast<int64_t>(i) * cols;
                        while (count < cols && !(ids[count] == -1 && std::isinf(ds[count]))) {
                            ++count;
                        }
                        auto* out_ids = new int64_t[std::max<int64_t>(count, 1)];
                        auto* out_d = new float[std::max<int64_t>(count, 1)];
                        std::copy(ids, ids + count, out_ids);
                        std::copy(ds, ds + count, out_d);
                        auto one = Dataset::Make();
                        one->NumElements(1)->Dim(count)->Ids(out_ids)->Distances(out_d)->Owner(true)->Statistics(stats);
                        batch[i]->result = one;
                    } else {
                        batch[i]->result = found;
                    }
                }
            }
        } catch (...) {
            for (PendingCall* c : batch) {
                c->error = std::current_exception();
            }
            release();
            throw;
        }
        release();
        return mine.result;
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

// Labels of a CalDistanceById call as inner ids (VSAG_AMD_INVALID_ID where the label is unknown).
std::vector<uint32_t>
inner_ids_of(const LabelMap& known, const int64_t* ids, int64_t total) {
    std::vector<uint32_t> inner(static_cast<size_t>(total));
    for (int64_t i = 0; i < total; ++i) {
        auto it = known.find(ids[i]);
        inner[i] = it == known.end() ? VSAG_AMD_INVALID_ID : it->second;
    }
    return inner;
}

// Distances of `rows` queries to `count` codes each, named by inner id, from a store (chunks of queries the device
// entry point takes at a time).
void
store_distances(SearchContext& ctx, const vsag_amd_store_t* store, const float* queries, int64_t rows, uint32_t dim,
                const std::vector<uint32_t>& inner, int64_t count, uint32_t scale, std::vector<float>& out) {
    out.assign(static_cast<size_t>(rows * count), -1.0F);
    if (count == 0) {
        return;
    }
    std::vector<uint32_t> scaled;
    const std::vector<uint32_t>* src = &inner;
    if (scale != 1) {
        scaled = inner;
        for (auto& v : scaled) {
            v = v == VSAG_AMD_INVALID_ID ? v : v * scale;
        }
        src = &scaled;
    }
    const int64_t chunk = 32768;
    for (int64_t r0 = 0; r0 < rows; r0 += chunk) {
        const int64_t nr = std::min(chunk, rows - r0);
        ctx.upload(ctx.queries, queries + r0 * dim, static_cast<size_t>(nr) * dim * 4);
        ctx.upload(ctx.cand_ids, src->data() + r0 * count, static_cast<size_t>(nr * count) * 4);
        ctx.out_d.reserve(static_cast<size_t>(nr * count) * 4);
        const size_t wsb = vsag_amd_store_distances_workspace_bytes(store, nr);
        ctx.workspace.reserve(wsb);
        dev(vsag_amd_store_distances(store, ctx.queries.as<float>(), nr, ctx.cand_ids.as<uint32_t>(),
                                     static_cast<uint32_t>(count), ctx.out_d.as<float>(), ctx.workspace.p, wsb, ctx.stream));
        ctx.download(out.data() + r0 * count, ctx.out_d.p, static_cast<size_t>(nr * count) * 4);
    }
}

// A posting list of pqfs codes as BucketDataCell keeps and serializes it (package_fastscan, bucket_datacell.h:943-966;
// PQFastScanQuantizer::Package32, pq_fastscan_quantizer.cpp:241-266): blocks of 32 codes, subspace i of a block in 16
// bytes, byte j / 2 holding the code of vector MAPPER[j] of the block in its low (even j) or high nibble; the last
// block is padded with zeros.  n plain codes of cs bytes -> ceil(n / 32) * 32 * cs bytes, and back.
constexpr int kPqMapper[32] = {0, 16, 8, 24, 1, 17, 9, 25, 2, 18, 10, 26, 3, 19, 11, 27,
                               4, 20, 12, 28, 5, 21, 13, 29, 6, 22, 14, 30, 7, 23, 15, 31};

void
pqfs_package_list(const uint8_t* codes, uint64_t n, uint32_t pq_dim, std::vector<uint8_t>& out) {
    const uint64_t cs = (pq_dim + 1) / 2, blocks = (n + 31) / 32;
    out.assign(blocks * 32 * cs, 0);
    for (uint64_t b = 0; b < blocks; ++b) {
        uint8_t* dst = out.data() + b * 32 * cs;
        for (uint32_t i = 0; i < pq_dim; ++i) {
            for (int j = 0; j < 32; ++j) {
                const uint64_t v = b * 32 + static_cast<uint64_t>(kPqMapper[j]);
                if (v >= n) {
                    continue;
                }
                const uint8_t nib = (codes[v * cs + i / 2] >> (4 * (i & 1))) & 15;
                dst[i * 16 + j / 2] |= static_cast<uint8_t>(nib << (4 * (j & 1)));
            }
        }
    }
}

void
pqfs_unpack_list(const uint8_t* packaged, uint64_t n, uint32_t pq_dim, uint8_t* codes) {
    const uint64_t cs = (pq_dim + 1) / 2;
    std::memset(codes, 0, n * cs);
    for (uint64_t b = 0; b * 32 < n; ++b) {
        const uint8_t* src = packaged + b * 32 * cs;
        for (uint32_t i = 0; i < pq_dim; ++i) {
            for (int j = 0; j < 32; ++j) {
                const uint64_t v = b * 32 + static_cast<uint64_t>(kPqMapper[j]);
                if (v >= n) {
                    continue;
                }
                const uint8_t nib = (src[i * 16 + j / 2] >> (4 * (j & 1))) & 15;
                codes[v * cs + i / 2] |= static_cast<uint8_t>(nib << (4 * (i & 1)));
            }
        }
    }
}

// FlattenDataCell::Serialize (src/datacell/flatten_datacell.h:481-497): [u32 total count][u32 capacity][u32 code size]
// [u64 bytes][codes by inner id][quantizer].  `rows`: the codes are fp32 rows kept outside a store.
void
write_flat_cell(Writer& w, const vsag_amd_store_t* store, const DevBuf* rows, const Quantizer& q, uint64_t total) {
    const uint64_t cs = q.code_size();
    w.obj(static_cast<uint32_t>(total));
    w.obj(static_cast<uint32_t>(std::max<uint64_t>(total, 800)));  // max_capacity_: never below its initial value
    w.obj(static_cast<uint32_t>(cs));
    w.obj(total * cs);
    const uint64_t step = std::max<uint64_t>(1, kIoChunkBytes / cs);
    std::vector<uint8_t> host(static_cast<size_t>(std::min(step, std::max<uint64_t>(total, 1)) * cs));
    DevBuf staged;
    for (uint64_t first = 0; first < total; first += step) {
        const uint64_t n = std::min(step, total - first);
        if (rows != nullptr) {
            dev(vsag_amd_memcpy_d2h(host.data(), rows->as<uint8_t>() + first * cs, n * cs, nullptr));
        } else {
            staged.reserve(n * cs);
            dev(vsag_amd_store_export_codes(store, first, n, staged.as<uint8_t>(), nullptr));
            dev(vsag_amd_memcpy_d2h(host.data(), staged.p, n * cs, nullptr));
        }
        w.write(host.data(), n * cs);
    }
    q.save(w);
}

// The cell back: the quantizer lies behind the codes, and the store is made from it, so the codes are read second.
// Returns the number of codes.
uint64_t
read_flat_cell(Reader& r, Quantizer& q, StoreHandle* store, DevBuf* rows) {
    const auto total = r.get<uint32_t>();
    (void)r.get<uint32_t>();
    const auto cs = r.get<uint32_t>();
    const auto bytes = r.get<uint64_t>();
    if (cs != q.code_size() || bytes < static_cast<uint64_t>(total) * cs) {
        throw VsagException(ErrorType::INVALID_ARGUMENT,
                            "the serialized codes (code size " + std::to_string(cs) + ", " + std::to_string(bytes) +
                                " bytes for " + std::to_string(total) + " codes) do not match the index (code size " +
                                std::to_string(q.code_size()) + ")");
    }
    const uint64_t codes_at = r.cursor();
    r.skip(bytes);
    q.load(r);
    const uint64_t behind = r.cursor();
    r.seek(codes_at);
    if (store != nullptr) {
        store->s = q.make_store();
        dev(vsag_amd_store_expect_stored_codes(store->s, 1));
    } else {
        rows->reserve(std::max<uint64_t>(static_cast<uint64_t>(total) * cs, 4));
    }
    const uint64_t step = std::max<uint64_t>(1, kIoChunkBytes / cs);
    std::vector<uint8_t> host(static_cast<size_t>(std::min<uint64_t>(step, std::max<uint32_t>(total, 1)) * cs));
    DevBuf staged;
    for (uint64_t first = 0; first < total; first += step) {
        const uint64_t n = std::min<uint64_t>(step, total - first);
        r.read(host.data(), n * cs);
        if (store != nullptr) {
            staged.reserve(n * cs);
            dev(vsag_amd_memcpy_h2d(staged.p, host.data(), n * cs, nullptr));
            dev(vsag_amd_store_append(store->s, staged.as<uint8_t>(), n, nullptr));
            dev(vsag_amd_stream_synchronize(nullptr));
        } else {
            dev(vsag_amd_memcpy_h2d(rows->as<uint8_t>() + first * cs, host.data(), n * cs, nullptr));
        }
    }
    if (store != nullptr) {
        dev(vsag_amd_store_expect_stored_codes(store->s, 0));
    }
    r.seek(behind);
    return total;
}

void
rebuild_label_map(const std::vector<int64_t>& labels, LabelMap& known) {
    known.clear();
    known.reserve(labels.size());
    for (size_t i = 0; i < labels.size(); ++i) {
        known.emplace(labels[i], static_cast<uint32_t>(i));
    }
}

DatasetPtr
empty_result(const std::string& stats = std::string()) {
    auto empty = Dataset::Make();
    empty->NumElements(1)->Dim(0);
    if (!stats.empty()) {
        empty->Statistics(stats);
    }
    return empty;
}

void
read_rabitq_params(const Json& index_param, Quantizer& q) {
    if (index_param.Contains("rabitq_bits_per_dim_query")) {
        q.rabitq_query_bits = static_cast<int>(index_param["rabitq_bits_per_dim_query"].GetInt());
    }
    if (q.kind == VSAG_AMD_KIND_RABITQ) {
        // RaBitQuantizerParameter::FromJson (rabitq_quantizer_parameter.cpp:30-112) and the constructor's checks
        // (rabitq_quantizer.cpp:67-100).
        CHECK_ARGUMENT(q.rabitq_query_bits == 4 || q.rabitq_query_bits == 32,
                       "currently, only support rabitq_bits_per_dim_query = 4 or 32, but got " +
                           std::to_string(q.rabitq_query_bits));
        if (index_param.Contains("rabitq_bits_per_dim_base")) {
            const int64_t bits = index_param["rabitq_bits_per_dim_base"].GetInt();
            CHECK_ARGUMENT(bits >= 1 && bits <= 8,
                           "currently, only support rabitq_bits_per_dim_base in [1, 8], but got " + std::to_string(bits));
            q.rabitq_base_bits = static_cast<int>(bits);
        }
        if (index_param.Contains("rabitq_version")) {
            const std::string version = index_param["rabitq_version"].GetString();
            CHECK_ARGUMENT(version == "standard" || version == "split" || version == "split_1bit_7bit",
                           "unsupported rabitq_version: " + version + ". Supported values are standard, split");
            // The split layout belongs to the flatten cell of the graph indexes (datacell/rabitq_split_datacell.h).
            CHECK_ARGUMENT(version == "standard", "rabitq_version=split is not supported on the GPU path");
        }
        CHECK_ARGUMENT(q.rabitq_query_bits != 4 || q.rabitq_base_bits == 1,
                       "not support num_bits_per_dim_query_ == 4 with num_bits_per_dim_base_ != 1");
        if (index_param.Contains("rabitq_error_rate")) {
            const double rate = index_param["rabitq_error_rate"].GetFloat();
            CHECK_ARGUMENT(std::isfinite(rate) && rate > 0.0,
                           "rabitq_error_rate must be finite and positive, got " + std::to_string(rate));
        }
        if (index_param.Contains("fast_encode_rabitq")) {
            q.rabitq_fast_encode = index_param["fast_encode_rabitq"].GetBool();
        }
        if (index_param.Contains("fast_encode_rabitq_rounds")) {
            CHECK_ARGUMENT(index_param["fast_encode_rabitq_rounds"].IsNumberInteger(),
                           "fast_encode_rabitq_rounds must be an integer");
            const int64_t rounds = index_param["fast_encode_rabitq_rounds"].GetInt();
            CHECK_ARGUMENT(rounds >= 1 && rounds <= 32,
                           "fast_encode_rabitq_rounds must be in [1, 32], but got " + std::to_string(rounds));
            q.rabitq_fast_rounds = static_cast<uint32_t>(rounds);
        }
        if (index_param.Contains("rabitq_use_fht")) {
            q.rabitq_use_fht = index_param["rabitq_use_fht"].GetBool();
        }
    }
}

// base_pq_dim (constants.cpp:197,211 -> PRODUCT_QUANTIZATION_DIM_KEY): the number of subspaces of a pqfs quantizer;
// the constructor of PQFastScanQuantizer rejects one that does not divide the dimension
// (pq_fastscan_quantizer.cpp:31-36).
void
read_pq_params(const Json& index_param, Quantizer& q) {
    if (q.kind != VSAG_AMD_KIND_PQFS) {
        return;
    }
    int64_t pq_dim = 1;
    if (index_param.Contains("base_pq_dim")) {
        pq_dim = index_param["base_pq_dim"].GetInt();
    }
    CHECK_ARGUMENT(pq_dim >= 1 && static_cast<int64_t>(q.dim) % pq_dim == 0,
                   "pq_dim(" + std::to_string(pq_dim) + ") does not divide evenly into dim(" + std::to_string(q.dim) + ")");
    CHECK_ARGUMENT(pq_dim <= 1024, "the GPU path supports base_pq_dim up to 1024, got " + std::to_string(pq_dim));
    q.pq_dim = static_cast<uint32_t>(pq_dim);
}

// ------------------------------------------------------------------------------------------- brute force
class BruteForce : public GpuIndex {
public:
    BruteForce(const CommonParam& common, const Json& index_param) {
        static const std::set<std::string> known = {
            "base_quantization_type", "base_io_type", "base_pq_dim", "base_file_path", "precise_quantization_type",
            "precise_io_type", "precise_file_path", "thread_count", "use_residual", "use_reorder",
            "use_attribute_filter", "rabitq_bits_per_dim_query", "rabitq_bits_per_dim_base", "rabitq_use_fht",
            "rabitq_version", "rabitq_error_rate", "fast_encode_rabitq", "fast_encode_rabitq_rounds"};
        reject_unknown_keys(index_param, known);
        q_.metric = common.metric;
        q_.dim = common.dim;
        q_.kind = VSAG_AMD_KIND_FP32;
        if (index_param.Contains("base_quantization_type")) {
            q_.kind = kind_from_name(index_param["base_quantization_type"].GetString());
        }
        read_rabitq_params(index_param, q_);
        read_pq_params(index_param, q_);
    }

    // BruteForce::Train (bruteforce.cpp:123-126): the quantizer of the codes is trained on the data.
    Expected<void>
    Train(const DatasetPtr& data) override {
        return safe_run([&]() {
            std::unique_lock<std::shared_mutex> lock(mutex_);
            check_base(data, q_.dim);
            if (q_.trained || data->GetNumElements() == 0) {
                return;
            }
            std::vector<int64_t> rows(static_cast<size_t>(data->GetNumElements()));
            for (size_t i = 0; i < rows.size(); ++i) {
                rows[i] = static_cast<int64_t>(i);
            }
            DevBuf x;
            upload_rows(data, rows, q_.dim, x);
            q_.train(x.as<float>(), rows.size());
        });
    }

    Expected<std::vector<int64_t>>
    Build(const DatasetPtr& base) override {
        return safe_call<std::vector<int64_t>>([&]() {
            std::unique_lock<std::shared_mutex> lock(mutex_);
            if (!labels_.empty()) {
                throw VsagException(ErrorType::BUILD_TWICE, "failed to build index: index is not empty");
            }
            return add_locked(base);
        });
    }

    Expected<std::vector<int64_t>>
    Add(const DatasetPtr& base) override {
        return safe_call<std::vector<int64_t>>([&]() {
            std::unique_lock<std::shared_mutex> lock(mutex_);
            return add_locked(base);
        });
    }

    int64_t
    GetNumElements() const override {
        std::shared_lock<std::shared_mutex> lock(mutex_);
        return static_cast<int64_t>(labels_.size());
    }

protected:
    uint32_t
    dimension() const override {
        return q_.dim;
    }

    DatasetPtr
    search(const DatasetPtr& query, int64_t k, const std::string& parameters, const SearchSpec& spec) const override {
        check_query(query, k, q_.dim);
        if (!parameters.empty()) {
            Json p = Json::Parse(parameters);  // {"parallelism": p}, optionally under "brute_force"
            CHECK_ARGUMENT(p.IsObject(), "search parameters must be a JSON object");
        }
        CHECK_ARGUMENT(spec.bucket_ids == nullptr, "bucket_ids_ is supported by the ivf index only");
        std::shared_lock<std::shared_mutex> lock(mutex_);
        const int64_t nq = query->GetNumElements();
        if (labels_.empty()) {
            return empty_result();
        }
        // One device scan returns at most 1024 results per query.  A range search, and a KnnSearch with a larger
        // k, run scan after scan for one query: what a scan returned is denied to the next one, so the rows come
        // out in ascending order.
        const bool looped = spec.range || k > kMaxDeviceK;
        CHECK_ARGUMENT(!spec.range || nq == 1, "range search takes one query");
        if (looped && nq > 1) {
            lock.unlock();
            return search_rows_one_by_one(query, k, parameters, spec);
        }
        auto ctx = pool_.acquire();
        ctx->upload(ctx->queries, query->GetFloat32Vectors(), static_cast<size_t>(nq) * q_.dim * 4);
        DenyMask mask;
        mask.init(*ctx, labels_, spec.valid, looped, 1);
        const vsag_amd_search_options_t opt = mask.options(*ctx, spec, 0.0F);
        // every stored vector once per query and scan
        SearchStats stats;
        stats.base_kind = q_.kind;
        const auto n = static_cast<int64_t>(labels_.size());
        if (!looped) {
            const auto kk = static_cast<uint32_t>(k);
            std::vector<uint32_t> ids;
            std::vector<float> dists;
            scan(*ctx, nq, kk, opt, ids, dists);
            stats.approximate = static_cast<uint64_t>(n) * static_cast<uint64_t>(nq);
            return pack_results(ids, dists, nq, k, labels_, stats.dump());
        }
        std::vector<std::pair<float, uint32_t>> row;
        int64_t remaining = spec.range ? (spec.limited_size > 0 ? spec.limited_size : n) : k;
        while (remaining > 0) {
            const auto kk = static_cast<uint32_t>(std::min<int64_t>({remaining, kMaxDeviceK, n}));
            std::vector<uint32_t> ids;
            std::vector<float> dists;
            scan(*ctx, 1, kk, opt, ids, dists);
            stats.approximate += static_cast<uint64_t>(n);
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
            mask.upload(*ctx);
        }
        if (row.empty()) {
            return empty_result(stats.dump());
        }
        return pack_row(row, labels_, stats.dump());
    }

    // BruteForce::CalDistanceById through InnerIndexInterface (inner_index_interface.cpp:448-609): the distance the
    // stored code gives, whatever calculate_precise_distance says (the index keeps one set of codes).
    DatasetPtr
    distances_by_id(const float* queries, int64_t rows, const int64_t* ids, int64_t count, bool /*precise*/,
                    int64_t topk) const override {
        std::shared_lock<std::shared_mutex> lock(mutex_);
        const std::vector<uint32_t> inner = inner_ids_of(known_, ids, rows * count);
        std::vector<float> dists(static_cast<size_t>(rows * count), -1.0F);
        if (count > 0 && store_.s != nullptr) {
            auto ctx = pool_.acquire();
            store_distances(*ctx, store_.s, queries, rows, q_.dim, inner, count, 1, dists);
        }
        return pack_distances(dists, inner, ids, rows, count, topk);
    }

    // BruteForceParameter::ToJson over InnerIndexParameter::ToJson (bruteforce_parameter.cpp:57-63,
    // inner_index_parameter.cpp:249-274).
    std::string
    index_param_json() const {
        return "{\"base_codes\":" + flatten_params_json(q_) +
               ",\"build_thread_count\":1,\"label_remap_type\":\"pg\",\"reorder_source\":\"precise\","
               "\"resize_increase_count_bit\":10,\"store_raw_vector\":false,\"train_sample_count\":65536,"
               "\"type\":\"brute_force\",\"use_attribute_filter\":false,\"use_reorder\":false}";
    }

    // BruteForce::Serialize (bruteforce.cpp:684-705): the codes' cell, the label table, the footer with basic_info.
    void
    save(Writer& w) const override {
        const uint64_t total = labels_.size();
        write_flat_cell(w, store_.s, nullptr, q_, total);
        w.vec(labels_);
        write_footer(w, "{\"_update_time\":\"1970-01-01 00:00:00\",\"basic_info\":{\"dim\":" + std::to_string(q_.dim) +
                            ",\"extra_info_size\":0,\"has_extra_info\":false,\"index_param\":" +
                            json_quoted(index_param_json()) + ",\"is_multi_vector\":false,\"total_count\":" +
                            std::to_string(total) + "}}");
    }

    // BruteForce::Deserialize (bruteforce.cpp:1001-1075), both the footer form and the older one that starts with
    // dim and count.
    void
    load(Reader& r) override {
        if (!labels_.empty()) {
            throw VsagException(ErrorType::INDEX_NOT_EMPTY, "failed to deserialize: index is not empty");
        }
        std::string metadata;
        uint64_t footer_bytes = 0;
        int64_t file_dim = q_.dim;
        uint64_t file_total = 0;
        const bool footer = read_footer(r, &metadata, &footer_bytes);
        if (footer) {
            const Json m = Json::Parse(metadata);
            if (m.Contains("_empty") && m["_empty"].GetBool()) {
                throw VsagException(ErrorType::INDEX_EMPTY, "index is empty");
            }
            CHECK_ARGUMENT(m.Contains("basic_info"), "the footer of the serialized index has no basic_info");
            const Json& info = m["basic_info"];
            file_dim = info["dim"].GetInt();
            file_total = static_cast<uint64_t>(info["total_count"].GetInt());
            if (info.Contains("extra_info_size")) {
                CHECK_ARGUMENT(info["extra_info_size"].GetInt() == 0, "BruteForce index extra_info_size not match");
            }
            if (info.Contains("index_param")) {
                // bruteforce.cpp:887-898 with BruteForceParameter::CheckCompatibility (bruteforce_parameter.cpp:65-73)
                const std::string text = info["index_param"].GetString();
                const Json file = Json::Parse(text);
                bool ok = inner_params_compatible(file, false, q_);
                if (ok && file.Contains("base_codes")) {
                    const Json& bc = file["base_codes"];
                    ok = (!bc.Contains("codes_type") || bc["codes_type"].GetString() == "flatten") &&
                         (!bc.Contains("quantization_params") ||
                          quantization_params_compatible(bc["quantization_params"], q_));
                }
                CHECK_ARGUMENT(ok, "BruteForce index parameter not match, current: " + index_param_json() + ", new: " + text);
            }
        } else {
            file_dim = r.get<int64_t>();
            file_total = r.get<uint64_t>();
        }
        CHECK_ARGUMENT(file_dim == static_cast<int64_t>(q_.dim), "the serialized index has dim " + std::to_string(file_dim) +
                                                                    ", this one " + std::to_string(q_.dim));
        Quantizer q = q_.blank();
        StoreHandle store;
        const uint64_t total = read_flat_cell(r, q, &store, nullptr);
        std::vector<int64_t> labels;
        r.vec(labels);
        if (total != file_total || labels.size() < total) {
            throw VsagException(ErrorType::INVALID_BINARY, "the serialized index holds " + std::to_string(total) +
                                                               " codes, " + std::to_string(labels.size()) +
                                                               " labels and a count of " + std::to_string(file_total));
        }
        labels.resize(total);
        q_.take(q);
        std::swap(store_.s, store.s);
        labels_.swap(labels);
        rebuild_label_map(labels_, known_);
    }

private:
    // One device scan of the uploaded queries; results copied to the host.
    void
    scan(SearchContext& ctx, int64_t nq, uint32_t kk, const vsag_amd_search_options_t& opt, std::vector<uint32_t>& ids,
         std::vector<float>& dists) const {
        ctx.out_ids.reserve(static_cast<size_t>(nq) * kk * 4);
        ctx.out_d.reserve(static_cast<size_t>(nq) * kk * 4);
        size_t wsb = vsag_amd_flat_scan_workspace_bytes(store_.s, nq, kk);
        ctx.workspace.reserve(wsb);
        dev(vsag_amd_flat_scan_topk_ex(store_.s, ctx.queries.as<float>(), nq, kk, &opt, ctx.out_ids.as<uint32_t>(),
                                       ctx.out_d.as<float>(), ctx.workspace.p, wsb, ctx.stream));
        ids.resize(static_cast<size_t>(nq) * kk);
        dists.resize(ids.size());
        ctx.download_later(ids.data(), ctx.out_ids.p, ids.size() * 4);
        ctx.download(dists.data(), ctx.out_d.p, dists.size() * 4);
    }

    std::vector<int64_t>
    add_locked(const DatasetPtr& base) {
        check_base(base, q_.dim);
        std::vector<int64_t> rows;
        std::vector<int64_t> failed = split_new_rows(base, known_, rows);
        if (rows.empty()) {
            return failed;
        }
        CHECK_ARGUMENT(labels_.size() + rows.size() < VSAG_AMD_INVALID_ID, "the index holds at most 2^32 - 2 vectors");
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
        }
        dev(vsag_amd_stream_synchronize(nullptr));
        // the labels are recorded once the device holds the vectors: a failed insert leaves the index as it was
        for (int64_t r : rows) {
            known_.emplace(base->GetIds()[r], static_cast<uint32_t>(labels_.size()));
            labels_.push_back(base->GetIds()[r]);
        }
        return failed;
    }

    Quantizer q_;
    StoreHandle store_;
    std::vector<int64_t> labels_;  // inner id -> label (LabelTable)
    LabelMap known_;
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
        pq_.metric = common.metric;
        pq_.dim = common.dim;
        if (index_param.Contains("base_quantization_type")) {
            q_.kind = kind_from_name(index_param["base_quantization_type"].GetString());
        }
        read_rabitq_params(index_param, q_);
        read_pq_params(index_param, q_);
        if (index_param.Contains("buckets_count")) {
            int64_t b = index_param["buckets_count"].GetInt();
            CHECK_ARGUMENT(b >= 1 && b <= (1 << 24), "buckets_count must be in [1, 2^24], got " + std::to_string(b));
            nlist_ = static_cast<uint32_t>(b);
        }
        if (index_param.Contains("use_reorder")) {
            use_reorder_ = index_param["use_reorder"].GetBool();
        }
        if (index_param.Contains("precise_quantization_type")) {
            pq_.kind = kind_from_name(index_param["precise_quantization_type"].GetString());
            CHECK_ARGUMENT(pq_.kind != VSAG_AMD_KIND_RABITQ, "precise_quantization_type must not be rabitq");
            // the reference's reorder asks a pqfs cell for single distances, which it refuses
            // (pq_fastscan_quantizer.cpp:158-164)
            CHECK_ARGUMENT(pq_.kind != VSAG_AMD_KIND_PQFS, "precise_quantization_type must not be pqfs");
        }
        if (index_param.Contains("precise_codes_layout")) {
            // "bucket" keeps the precise codes list by list instead of in one array (ivf.cpp:441-455); the distances are
            // the same, and here both are one array addressed by inner id.
            const std::string layout = index_param["precise_codes_layout"].GetString();
            CHECK_ARGUMENT(layout == "flat" || layout == "bucket", "precise_codes_layout must be flat or bucket");
            CHECK_ARGUMENT(layout == "flat" || use_reorder_, "precise_codes_layout=bucket requires use_reorder=true");
        }
        if (index_param.Contains("ivf_train_type")) {
            const std::string t = index_param["ivf_train_type"].GetString();
            CHECK_ARGUMENT(t == "kmeans" || t == "random", "ivf_train_type must be kmeans or random, got " + t);
            train_random_ = t == "random";
        }
        if (index_param.Contains("buckets_per_data")) {
            // ivf_parameter.cpp:36-46
            const int64_t b = index_param["buckets_per_data"].GetInt();
            CHECK_ARGUMENT(b >= 1 && b <= static_cast<int64_t>(nlist_),
                           "buckets_per_data must be in [1, buckets_count], got " + std::to_string(b));
            CHECK_ARGUMENT(b <= 64, "the GPU path supports buckets_per_data up to 64");
            bpd_ = static_cast<uint32_t>(b);
        }
        if (index_param.Contains("use_residual")) {
            use_residual_ = index_param["use_residual"].GetBool();
        }
        if (index_param.Contains("partition_strategy_type")) {
            CHECK_ARGUMENT(index_param["partition_strategy_type"].GetString() == "ivf",
                           "the GPU path supports the nearest-centroid partition strategy only");
        }
        if (index_param.Contains("graph_build_threshold")) {
            CHECK_ARGUMENT(index_param["graph_build_threshold"].GetInt() <= 0,
                           "the GPU path scans lists flat: graph_build_threshold must be 0");
        }
        // ivf_parameter.cpp:88-98: default max(65536, 64 * buckets_count), at least 512.
        train_sample_count_ = std::max<int64_t>(65536, 64LL * nlist_);
        if (index_param.Contains("train_sample_count")) {
            train_sample_count_ = index_param["train_sample_count"].GetInt();
            CHECK_ARGUMENT(train_sample_count_ >= 512, "train_sample_count must be at least 512");
        }
    }

    // IVF::Train (ivf.cpp:564-588).
    Expected<void>
    Train(const DatasetPtr& data) override {
        return safe_run([&]() {
            std::unique_lock<std::shared_mutex> lock(mutex_);
            check_base(data, q_.dim);
            if (trained_) {
                return;
            }
            std::vector<int64_t> rows(static_cast<size_t>(data->GetNumElements()));
            for (size_t i = 0; i < rows.size(); ++i) {
                rows[i] = static_cast<int64_t>(i);
            }
            train_locked(data, rows, nullptr);
        });
    }

    // IVF::Build = Train + Add (ivf.cpp:547-562).
    Expected<std::vector<int64_t>>
    Build(const DatasetPtr& base) override {
        return safe_call<std::vector<int64_t>>([&]() {
            std::unique_lock<std::shared_mutex> lock(mutex_);
            if (!labels_.empty()) {
                throw VsagException(ErrorType::BUILD_TWICE, "failed to build index: index is not empty");
            }
            return add_locked(base, true);
        });
    }

    Expected<std::vector<int64_t>>
    Add(const DatasetPtr& base) override {
        return safe_call<std::vector<int64_t>>([&]() {
            std::unique_lock<std::shared_mutex> lock(mutex_);
            return add_locked(base, false);
        });
    }

    int64_t
    GetNumElements() const override {
        std::shared_lock<std::shared_mutex> lock(mutex_);
        return static_cast<int64_t>(labels_.size());
    }

protected:
    uint32_t
    dimension() const override {
        return q_.dim;
    }

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
        const bool disable_scan = ivf.Contains("disable_bucket_scan") && ivf["disable_bucket_scan"].GetBool();
        const int64_t nq = query->GetNumElements();
        if (spec.bucket_ids != nullptr) {
            // IVF::SearchWithRequest (ivf.cpp:2076-2110)
            CHECK_ARGUMENT(static_cast<int64_t>(spec.bucket_ids->size()) == nq,
                           "bucket_ids_ size must match the number of query vectors; got " +
                               std::to_string(spec.bucket_ids->size()) + " bucket lists for " + std::to_string(nq) +
                               " queries");
            CHECK_ARGUMENT(!disable_scan, "bucket_ids_ is incompatible with disable_bucket_scan mode");
            for (size_t qi = 0; qi < spec.bucket_ids->size(); ++qi) {
                const auto& ids = (*spec.bucket_ids)[qi];
                CHECK_ARGUMENT(!ids.empty(), "bucket_ids_[" + std::to_string(qi) +
                                                 "] must not be empty; use empty outer vector for default routing");
                std::set<int64_t> seen;
                for (int64_t id : ids) {
                    CHECK_ARGUMENT(id >= 0 && id < static_cast<int64_t>(nlist_),
                                   "bucket_id " + std::to_string(id) + " out of range [0, " + std::to_string(nlist_) + ")");
                    CHECK_ARGUMENT(seen.insert(id).second, "duplicate bucket_id " + std::to_string(id));
                }
            }
        }

        std::shared_lock<std::shared_mutex> lock(mutex_);
        check_usable();
        if (labels_.empty()) {
            return empty_result();
        }
        const auto n = static_cast<int64_t>(labels_.size());
        uint32_t nprobe = static_cast<uint32_t>(std::min<int64_t>(scan, nlist_));  // ivf.cpp:1573-1574
        const bool reorder = use_reorder_ && enable_reorder;
        if (reorder) {
            CHECK_ARGUMENT(factor > 0.0F, "factor must be positive when use_reorder is true");
        }
        int64_t kcand = k;
        if (reorder && !spec.range) {
            kcand = std::max<int64_t>(static_cast<int64_t>(factor * static_cast<float>(k)), 1);  // ivf.cpp:2316
        }
        // One device scan returns at most 1024 candidates per query; more (and every range search) run scan
        // after scan for one query, each denied what the earlier ones returned.  With buckets_per_data = b a vector
        // has b postings, so a scan asks for b times the candidates (ivf.cpp:1722-1730).
        const bool looped = spec.range || kcand * bpd_ > kMaxDeviceK;
        CHECK_ARGUMENT(!spec.range || nq == 1, "range search takes one query");
        if (looped && nq > 1) {
            lock.unlock();
            return search_rows_one_by_one(query, k, parameters, spec);
        }

        auto lease = pool_.acquire();
        SearchContext& ctx = *lease;
        ctx.upload(ctx.queries, query->GetFloat32Vectors(), static_cast<size_t>(nq) * q_.dim * 4);
        SearchStats stats;
        stats.base_kind = q_.kind;
        stats.precise_kind = pq_.kind;
        if (spec.bucket_ids != nullptr) {
            // the caller names the lists (ivf.cpp:1702-1706); shorter rows are padded with "no list"
            size_t widest = 0;
            for (const auto& ids : *spec.bucket_ids) {
                widest = std::max(widest, ids.size());
            }
            nprobe = static_cast<uint32_t>(widest);
            std::vector<int32_t> padded(static_cast<size_t>(nq) * nprobe, -1);
            for (int64_t qi = 0; qi < nq; ++qi) {
                const auto& ids = (*spec.bucket_ids)[qi];
                for (size_t j = 0; j < ids.size(); ++j) {
                    padded[qi * nprobe + j] = static_cast<int32_t>(ids[j]);
                }
            }
            ctx.upload(ctx.buckets, padded.data(), padded.size() * 4);
        } else {
            // 1. route (exact nearest centroids)
            ctx.buckets.reserve(static_cast<size_t>(nq) * nprobe * 4);
            ctx.bucket_d.reserve(static_cast<size_t>(nq) * nprobe * 4);
            const size_t wsb = vsag_amd_ivf_route_workspace_bytes(centroid_store_.s, nq, nprobe);
            ctx.workspace.reserve(wsb);
            dev(vsag_amd_ivf_route(centroid_store_.s, ctx.queries.as<float>(), nq, nprobe, ctx.buckets.as<int32_t>(),
                                   ctx.bucket_d.as<float>(), ctx.workspace.p, wsb, ctx.stream));
            stats.routing = static_cast<uint64_t>(nq) * nlist_;
        }
        if (disable_scan && !spec.range) {
            // routing only: bucket ids + centroid distances (ivf.cpp:1589-1660)
            std::vector<uint32_t> ids(static_cast<size_t>(nq) * nprobe);
            std::vector<float> dists(ids.size());
            ctx.download_later(ids.data(), ctx.buckets.p, ids.size() * 4);
            ctx.download(dists.data(), ctx.bucket_d.p, dists.size() * 4);
            std::vector<int64_t> identity(nlist_);
            for (uint32_t i = 0; i < nlist_; ++i) {
                identity[i] = i;
            }
            return pack_results(ids, dists, nq, nprobe, identity, stats.dump());
        }
        const uint64_t probed = probed_codes(ctx, nq, nprobe);
        DenyMask mask;
        mask.init(ctx, labels_, spec.valid, looped, bpd_);
        // FlatBucketSearcher compares against radius + THRESHOLD_ERROR (flat_bucket_searcher.cpp:121,
        // impl/searcher/basic_searcher.h:39).
        const vsag_amd_search_options_t opt = mask.options(ctx, spec, 2e-6F);

        if (!looped) {
            // 2. scan the probed lists; 3. exact rerank, best min(k, candidates) kept (flatten_reorder.cpp:77)
            const auto kc = static_cast<uint32_t>(kcand * bpd_);
            const int64_t kout = reorder ? std::min<int64_t>(k, kcand) : kcand;
            scan_lists(ctx, nq, nprobe, kc, opt);
            stats.approximate = probed;
            std::vector<uint32_t> ids;
            std::vector<float> dists;
            if (bpd_ == 1 && reorder && pq_.kind == VSAG_AMD_KIND_FP32) {
                // the whole batch stays on the device
                ctx.out_ids.reserve(static_cast<size_t>(nq) * kout * 4);
                ctx.out_d.reserve(static_cast<size_t>(nq) * kout * 4);
                dev(vsag_amd_rerank_fp32(raw_.as<float>(), labels_.size(), q_.dim, q_.metric, ctx.queries.as<float>(), nq,
                                         ctx.cand_ids.as<uint32_t>(), kc, static_cast<uint32_t>(kout),
                                         ctx.out_ids.as<uint32_t>(), ctx.out_d.as<float>(), ctx.stream));
                fetch(ctx, ctx.out_ids, ctx.out_d, static_cast<size_t>(nq) * kout, ids, dists);
                stats.rerank = static_cast<uint64_t>(nq) * kc;  // at most: lists may hold fewer candidates
                return pack_results(ids, dists, nq, kout, labels_, stats.dump());
            }
            fetch(ctx, ctx.cand_ids, ctx.cand_d, static_cast<size_t>(nq) * kc, ids, dists);
            if (bpd_ > 1) {
                merge_postings(ids, dists, nq, kc, static_cast<uint32_t>(kcand));
            }
            if (reorder) {
                std::vector<uint32_t> best;
                std::vector<float> best_d;
                stats.rerank = rerank(ctx, nq, ids, static_cast<uint32_t>(kcand), static_cast<uint32_t>(kout), best, best_d);
                return pack_results(best, best_d, nq, kout, labels_, stats.dump());
            }
            return pack_results(ids, dists, nq, kout, labels_, stats.dump());
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
        std::unordered_set<uint32_t> seen;
        int64_t remaining = want;
        while (remaining > 0) {
            const auto kc = static_cast<uint32_t>(
                std::min<int64_t>({remaining * bpd_, kMaxDeviceK, n * static_cast<int64_t>(bpd_)}));
            scan_lists(ctx, 1, nprobe, kc, opt);
            stats.approximate += probed;
            std::vector<uint32_t> ids;
            std::vector<float> dists;
            fetch(ctx, ctx.cand_ids, ctx.cand_d, kc, ids, dists);
            uint32_t got = 0;
            while (got < kc && ids[got] != VSAG_AMD_INVALID_ID) {
                // ascending: the first posting of a vector carries its smallest distance (ivf.cpp:1799-1812)
                const uint32_t origin = ids[got] / bpd_;
                if (remaining > 0 && seen.insert(origin).second) {
                    row.emplace_back(dists[got], origin);
                    mask.deny(origin);
                    --remaining;
                }
                ++got;
            }
            if (got < kc) {
                break;
            }
            mask.upload(ctx);
        }
        if (reorder && !row.empty()) {
            // exact distances of everything gathered, a device call per 1024 candidates
            std::vector<std::pair<float, uint32_t>> exact;
            for (size_t i0 = 0; i0 < row.size(); i0 += kMaxDeviceK) {
                const auto m = static_cast<uint32_t>(std::min<size_t>(kMaxDeviceK, row.size() - i0));
                std::vector<uint32_t> cand(m);
                for (uint32_t i = 0; i < m; ++i) {
                    cand[i] = row[i0 + i].second;
                }
                std::vector<uint32_t> best;
                std::vector<float> best_d;
                stats.rerank += rerank(ctx, 1, cand, m, m, best, best_d);
                for (uint32_t i = 0; i < m && best[i] != VSAG_AMD_INVALID_ID; ++i) {
                    exact.emplace_back(best_d[i], best[i]);
                }
            }
            std::sort(exact.begin(), exact.end());
            if (static_cast<int64_t>(exact.size()) > keep) {
                exact.resize(static_cast<size_t>(keep));
            }
            row.swap(exact);
        }
        if (row.empty()) {
            return empty_result(stats.dump());
        }
        return pack_row(row, labels_, stats.dump());
    }

    // IVF::CalDistanceById (ivf.cpp:2429-2508): the precise codes when the index reorders and the caller asks for
    // precise distances, else the codes of the lists (the first posting of the vector, ivf.cpp:670-675).
    DatasetPtr
    distances_by_id(const float* queries, int64_t rows, const int64_t* ids, int64_t count, bool precise,
                    int64_t topk) const override {
        std::shared_lock<std::shared_mutex> lock(mutex_);
        check_usable();
        const std::vector<uint32_t> inner = inner_ids_of(known_, ids, rows * count);
        std::vector<float> dists(static_cast<size_t>(rows * count), -1.0F);
        if (count > 0 && !labels_.empty()) {
            auto lease = pool_.acquire();
            SearchContext& ctx = *lease;
            if (use_reorder_ && precise && pq_.kind == VSAG_AMD_KIND_FP32) {
                const int64_t chunk = 32768;
                for (int64_t r0 = 0; r0 < rows; r0 += chunk) {
                    const int64_t nr = std::min(chunk, rows - r0);
                    ctx.upload(ctx.queries, queries + r0 * q_.dim, static_cast<size_t>(nr) * q_.dim * 4);
                    ctx.upload(ctx.cand_ids, inner.data() + r0 * count, static_cast<size_t>(nr * count) * 4);
                    ctx.out_d.reserve(static_cast<size_t>(nr * count) * 4);
                    dev(vsag_amd_rows_distances_fp32(raw_.as<float>(), labels_.size(), q_.dim, q_.metric,
                                                     ctx.queries.as<float>(), nr, ctx.cand_ids.as<uint32_t>(),
                                                     static_cast<uint32_t>(count), ctx.out_d.as<float>(), ctx.stream));
                    ctx.download(dists.data() + r0 * count, ctx.out_d.p, static_cast<size_t>(nr * count) * 4);
                }
            } else if (use_reorder_ && precise) {
                store_distances(ctx, precise_.s, queries, rows, q_.dim, inner, count, 1, dists);
            } else {
                store_distances(ctx, lists_.s, queries, rows, q_.dim, inner, count, bpd_, dists);
            }
        }
        return pack_distances(dists, inner, ids, rows, count, topk);
    }

    // IVF::Serialize (ivf.cpp:990-1057): the cells "bucket", "partition_strategy", "label_table" and "reorder_codes",
    // their offsets and sizes in the footer next to basic_info.  The bucket cell is BucketDataCell::Serialize
    // (bucket_datacell.h:892-904).  The partition cell starts like IVFPartitionStrategy::Serialize
    // (ivf_partition_strategy.h:76-80); behind that the reference writes the image of its router graph, this index
    // (which routes exactly) a tag and the centroids -- load() reads both, the reference reads only its own.
    static constexpr uint64_t kCentroidTag = 0x52444D4147415356ULL;  // "VSAGAMDR"

    void
    save(Writer& w) const override {
        check_usable();
        std::string offsets = "{", sizes = "{";
        auto cell = [&](const char* name, uint64_t begin) {
            offsets += std::string(offsets.size() > 1 ? "," : "") + "\"" + name + "\":" + std::to_string(begin);
            sizes += std::string(sizes.size() > 1 ? "," : "") + "\"" + name + "\":" + std::to_string(w.cursor() - begin);
        };
        const uint64_t postings = labels_.size() * bpd_;
        const uint64_t cs = q_.code_size();
        // bucket
        uint64_t begin = w.cursor();
        w.obj(static_cast<int32_t>(nlist_));
        w.obj(static_cast<uint32_t>(cs));
        q_.save(w);
        std::vector<uint32_t> list_sizes(nlist_, 0);
        std::vector<uint8_t> codes;
        std::vector<uint32_t> ids;
        std::vector<float> bias;
        const bool with_bias = use_residual_ && q_.metric == VSAG_AMD_METRIC_L2;
        if (postings > 0) {
            dev(vsag_amd_store_list_sizes(lists_.s, list_sizes.data(), nlist_));
            DevBuf dcodes, dids, dbias;
            dcodes.reserve(postings * cs);
            dids.reserve(postings * 4);
            if (with_bias) {
                dbias.reserve(postings * 4);
            }
            dev(vsag_amd_store_export_lists(lists_.s, dcodes.as<uint8_t>(), dids.as<uint32_t>(),
                                            with_bias ? dbias.as<float>() : nullptr, nullptr));
            codes.resize(postings * cs);
            ids.resize(postings);
            dev(vsag_amd_memcpy_d2h(codes.data(), dcodes.p, codes.size(), nullptr));
            dev(vsag_amd_memcpy_d2h(ids.data(), dids.p, ids.size() * 4, nullptr));
            if (with_bias) {
                bias.resize(postings);
                dev(vsag_amd_memcpy_d2h(bias.data(), dbias.p, bias.size() * 4, nullptr));
            }
        }
        uint64_t at = 0;
        std::vector<uint8_t> packaged;
        for (uint32_t l = 0; l < nlist_; ++l) {
            const uint64_t n = list_sizes[l];
            if (q_.kind == VSAG_AMD_KIND_PQFS) {
                pqfs_package_list(codes.data() + at * cs, n, q_.pq_dim, packaged);
                w.obj(static_cast<uint64_t>(packaged.size()));
                w.write(packaged.data(), packaged.size());
            } else {
                w.obj(n * cs);
                w.write(codes.data() + at * cs, n * cs);
            }
            w.obj(n);
            w.write(ids.data() + at, n * 4);
            if (use_residual_) {
                const uint64_t nb = with_bias ? n : 0;
                w.obj(nb);
                if (nb > 0) {
                    w.write(bias.data() + at, nb * 4);
                }
            }
            at += n;
        }
        w.vec(list_sizes);
        cell("bucket", begin);
        // partition_strategy
        begin = w.cursor();
        w.obj(static_cast<uint8_t>(trained_ ? 1 : 0));
        w.obj(static_cast<int32_t>(nlist_));
        w.obj(static_cast<int64_t>(q_.dim));
        w.obj(kCentroidTag);
        std::vector<float> centroids(trained_ ? static_cast<size_t>(nlist_) * q_.dim : 0);
        if (!centroids.empty()) {
            dev(vsag_amd_memcpy_d2h(centroids.data(), centroids_.p, centroids.size() * 4, nullptr));
        }
        w.vec(centroids);
        cell("partition_strategy", begin);
        // label_table
        begin = w.cursor();
        w.vec(labels_);
        cell("label_table", begin);
        if (use_reorder_) {
            begin = w.cursor();
            if (pq_.kind == VSAG_AMD_KIND_FP32) {
                Quantizer fp = pq_.blank();
                fp.trained = trained_;
                write_flat_cell(w, nullptr, &raw_, fp, labels_.size());
            } else {
                write_flat_cell(w, precise_.s, nullptr, pq_, labels_.size());
            }
            cell("reorder_codes", begin);
        }
        write_footer(w, "{\"_update_time\":\"1970-01-01 00:00:00\",\"basic_info\":{\"data_type\":0,\"dim\":" +
                            std::to_string(q_.dim) + ",\"extra_info_size\":0,\"index_param\":" +
                            json_quoted(index_param_json()) + ",\"is_trained\":" +
                            (trained_ ? "true" : "false") + ",\"metric\":" + std::to_string(q_.metric) +
                            ",\"total_elements\":" + std::to_string(labels_.size()) + ",\"use_reorder\":" +
                            (use_reorder_ ? "true" : "false") + "},\"datacell_offsets\":" + offsets +
                            "},\"datacell_sizes\":" + sizes + "}}");
    }

    // IVFParameter::ToJson over InnerIndexParameter::ToJson (ivf_parameter.cpp:121-132, inner_index_parameter.cpp:249-274)
    // with BucketDataCellParameter::ToJson (bucket_datacell_parameter.cpp:48-55) and
    // IVFPartitionStrategyParameters::ToJson (ivf_partition_strategy_parameter.cpp:69-88).
    std::string
    index_param_json() const {
        std::string s = "{\"build_thread_count\":1,\"buckets_params\":{\"buckets_count\":" + std::to_string(nlist_) +
                        ",\"io_params\":{\"type\":\"memory_io\"},\"quantization_params\":" + quantization_params_json(q_) +
                        ",\"use_residual\":" + (use_residual_ ? "true" : "false") + "},\"buckets_per_data\":" +
                        std::to_string(bpd_) + ",\"graph_build_threshold\":0,\"label_remap_type\":\"pg\","
                        "\"partition_strategy\":{\"ivf_train_type\":\"" + (train_random_ ? "random" : "kmeans") +
                        "\",\"partition_strategy_type\":\"ivf\",\"route_ef_construction\":300,\"route_max_degree\":64}";
        if (use_reorder_) {
            s += ",\"precise_codes\":" + flatten_params_json(pq_);
        }
        s += ",\"precise_codes_layout\":\"flat\",\"reorder_source\":\"precise\",\"store_raw_vector\":false,"
             "\"train_sample_count\":" + std::to_string(train_sample_count_) +
             ",\"type\":\"ivf\",\"use_attribute_filter\":false,\"use_reorder\":" + (use_reorder_ ? "true" : "false") + "}";
        return s;
    }

    // IVFParameter::CheckCompatibility (ivf_parameter.cpp:133-148) against the parameters a file carries.
    bool
    index_param_compatible(const Json& file) const {
        if (!inner_params_compatible(file, use_reorder_, pq_)) {
            return false;
        }
        if (file.Contains("precise_codes_layout") && file["precise_codes_layout"].GetString() != "flat") {
            return false;
        }
        if (file.Contains("buckets_per_data") && file["buckets_per_data"].GetInt() != static_cast<int64_t>(bpd_)) {
            return false;
        }
        if (file.Contains("graph_build_threshold") && file["graph_build_threshold"].GetInt() != 0) {
            return false;
        }
        if (file.Contains("buckets_params")) {
            const Json& bp = file["buckets_params"];
            if (bp.Contains("quantization_params") && !quantization_params_compatible(bp["quantization_params"], q_)) {
                return false;
            }
            if (bp.Contains("buckets_count") && bp["buckets_count"].GetInt() != static_cast<int64_t>(nlist_)) {
                return false;
            }
            if (bp.Contains("use_residual") && bp["use_residual"].GetBool() != use_residual_) {
                return false;
            }
        }
        if (file.Contains("partition_strategy")) {
            const Json& ps = file["partition_strategy"];
            if (ps.Contains("partition_strategy_type") && ps["partition_strategy_type"].GetString() != "ivf") {
                return false;
            }
            if ((ps.Contains("route_max_degree") && ps["route_max_degree"].GetInt() != 64) ||
                (ps.Contains("route_ef_construction") && ps["route_ef_construction"].GetInt() != 300)) {
                return false;
            }
        }
        return true;
    }

    // IVF::Deserialize (ivf.cpp:1429-1530), footer form.
    void
    load(Reader& r) override {
        if (!labels_.empty() || trained_) {
            throw VsagException(ErrorType::INDEX_NOT_EMPTY, "failed to deserialize: index is not empty");
        }
        std::string metadata;
        uint64_t footer_bytes = 0;
        if (!read_footer(r, &metadata, &footer_bytes)) {
            throw VsagException(ErrorType::INVALID_BINARY, "the serialized ivf index has no footer");
        }
        const Json m = Json::Parse(metadata);
        if (m.Contains("_empty") && m["_empty"].GetBool()) {
            return;
        }
        CHECK_ARGUMENT(m.Contains("basic_info") && m.Contains("datacell_offsets") && m.Contains("datacell_sizes"),
                       "the footer of the serialized index lacks basic_info or the cells' offsets and sizes");
        const Json& info = m["basic_info"];
        const Json& offsets = m["datacell_offsets"];
        const auto total = static_cast<uint64_t>(info["total_elements"].GetInt());
        CHECK_ARGUMENT(info["dim"].GetInt() == static_cast<int64_t>(q_.dim), "the serialized index has another dim");
        CHECK_ARGUMENT(!info.Contains("metric") || info["metric"].GetInt() == q_.metric,
                       "the serialized index has another metric");
        CHECK_ARGUMENT(info["use_reorder"].GetBool() == use_reorder_,
                       "the serialized index and this one differ in use_reorder");
        if (info.Contains("index_param")) {  // ivf.cpp:1201-1208
            const std::string text = info["index_param"].GetString();
            CHECK_ARGUMENT(index_param_compatible(Json::Parse(text)),
                           "IVF index parameter not match, current: " + index_param_json() + ", new: " + text);
        }
        CHECK_ARGUMENT(total * bpd_ < VSAG_AMD_INVALID_ID, "the serialized index holds too many postings");
        for (const char* name : {"bucket", "partition_strategy", "label_table"}) {
            CHECK_ARGUMENT(offsets.Contains(name), std::string("the serialized index has no cell ") + name);
        }
        const bool file_trained = info["is_trained"].GetBool();

        // partition_strategy first: the lists of a residual index need its centroids
        r.seek(static_cast<uint64_t>(offsets["partition_strategy"].GetInt()));
        (void)r.get<uint8_t>();
        const auto file_lists = r.get<int32_t>();
        const auto file_dim = r.get<int64_t>();
        CHECK_ARGUMENT(file_lists == static_cast<int32_t>(nlist_) && file_dim == static_cast<int64_t>(q_.dim),
                       "the serialized partition has " + std::to_string(file_lists) + " buckets of dim " +
                           std::to_string(file_dim) + ", this index " + std::to_string(nlist_) + " of dim " +
                           std::to_string(q_.dim));
        std::vector<float> centroids;
        if (r.get<uint64_t>() == kCentroidTag) {
            r.vec(centroids);
        } else {
            r.seek(r.cursor() - 8);
            read_router_image(r, centroids);
        }
        CHECK_ARGUMENT(!file_trained || centroids.size() == static_cast<size_t>(nlist_) * q_.dim,
                       "the serialized partition does not hold one centroid per bucket");
        DevBuf centroids_dev;
        StoreHandle router;
        if (file_trained) {
            centroids_dev.reserve(centroids.size() * 4);
            dev(vsag_amd_memcpy_h2d(centroids_dev.p, centroids.data(), centroids.size() * 4, nullptr));
            Quantizer cq;
            cq.kind = VSAG_AMD_KIND_FP32;
            cq.metric = q_.metric;
            cq.dim = q_.dim;
            router.s = cq.make_store();
            dev(vsag_amd_store_expect_stored_codes(router.s, 1));  // cosine: unit vectors already
            dev(vsag_amd_store_append(router.s, centroids_dev.as<uint8_t>(), nlist_, nullptr));
            dev(vsag_amd_store_expect_stored_codes(router.s, 0));
        }

        // bucket
        r.seek(static_cast<uint64_t>(offsets["bucket"].GetInt()));
        const auto buckets = r.get<int32_t>();
        const auto cs = r.get<uint32_t>();
        CHECK_ARGUMENT(buckets == static_cast<int32_t>(nlist_) && cs == q_.code_size(),
                       "the serialized lists (" + std::to_string(buckets) + " of code size " + std::to_string(cs) +
                           ") do not match the index (" + std::to_string(nlist_) + " of code size " +
                           std::to_string(q_.code_size()) + ")");
        Quantizer q = q_.blank();
        q.load(r);
        // the sizes lie behind the lists: a first walk finds them, the second one reads the lists
        const uint64_t lists_at = r.cursor();
        for (uint32_t l = 0; l < nlist_; ++l) {
            r.skip(r.get<uint64_t>());
            r.skip(r.get<uint64_t>() * 4);
            if (use_residual_) {
                r.skip(r.get<uint64_t>() * 4);
            }
        }
        std::vector<uint32_t> list_sizes;
        r.vec(list_sizes);
        CHECK_ARGUMENT(list_sizes.size() == nlist_, "serialized bucket size vector does not match bucket count");
        uint64_t postings = 0;
        for (uint32_t n : list_sizes) {
            postings += n;
        }
        if (postings != total * bpd_) {
            throw VsagException(ErrorType::INVALID_BINARY, "the lists hold " + std::to_string(postings) + " codes for " +
                                                               std::to_string(total) + " vectors with buckets_per_data " +
                                                               std::to_string(bpd_));
        }
        const bool with_bias = use_residual_ && q_.metric == VSAG_AMD_METRIC_L2;
        std::vector<uint8_t> codes(postings * cs);
        std::vector<int32_t> bucket_of(postings, -1);
        std::vector<float> bias(with_bias ? postings : 0, 0.0F);
        std::vector<uint8_t> list_codes;
        std::vector<uint32_t> list_ids;
        std::vector<float> list_bias;
        r.seek(lists_at);
        for (uint32_t l = 0; l < nlist_; ++l) {
            const uint64_t n = list_sizes[l];
            const auto bytes = r.get<uint64_t>();
            if (bytes < n * cs) {
                throw VsagException(ErrorType::INVALID_BINARY, "a serialized list is shorter than its size");
            }
            list_codes.resize(n * cs);
            if (q_.kind == VSAG_AMD_KIND_PQFS) {
                // whole blocks of 32 codes in the fast-scan order
                const uint64_t padded = (n + 31) / 32 * 32 * cs;
                if (bytes < padded) {
                    throw VsagException(ErrorType::INVALID_BINARY, "a serialized pqfs list is not made of whole blocks");
                }
                std::vector<uint8_t> packaged(padded);
                r.read(packaged.data(), padded);
                r.skip(bytes - padded);
                pqfs_unpack_list(packaged.data(), n, q_.pq_dim, list_codes.data());
            } else {
                r.read(list_codes.data(), n * cs);
                r.skip(bytes - n * cs);
            }
            r.vec(list_ids);
            if (list_ids.size() < n) {
                throw VsagException(ErrorType::INVALID_BINARY,
                                    "serialized bucket " + std::to_string(l) + " inner id count is smaller than bucket size");
            }
            if (use_residual_) {
                r.vec(list_bias);
                if (with_bias && list_bias.size() < n) {
                    throw VsagException(ErrorType::INVALID_BINARY, "a serialized list lacks residual bias values");
                }
            }
            for (uint64_t i = 0; i < n; ++i) {
                const uint32_t id = list_ids[i];
                if (id >= postings || bucket_of[id] != -1) {
                    throw VsagException(ErrorType::INVALID_BINARY, "the serialized lists name inner id " +
                                                                       std::to_string(id) + " twice or out of range");
                }
                bucket_of[id] = static_cast<int32_t>(l);
                std::memcpy(codes.data() + static_cast<uint64_t>(id) * cs, list_codes.data() + i * cs, cs);
                if (with_bias) {
                    bias[id] = list_bias[i];
                }
            }
        }
        StoreHandle lists;
        if (file_trained) {
            lists.s = q.make_store();
            dev(vsag_amd_store_expect_stored_codes(lists.s, 1));
            if (use_residual_) {
                dev(vsag_amd_store_set_residual(lists.s, centroids_dev.as<float>(), nlist_, nullptr));
            }
            dev(vsag_amd_store_set_lists(lists.s, nullptr, nullptr, 0, nlist_, nullptr));
            const uint64_t step = std::max<uint64_t>(1, kIoChunkBytes / cs);
            DevBuf dcodes, dlabels, dbias;
            for (uint64_t first = 0; first < postings; first += step) {
                const uint64_t n = std::min(step, postings - first);
                dcodes.reserve(n * cs);
                dlabels.reserve(n * 4);
                dev(vsag_amd_memcpy_h2d(dcodes.p, codes.data() + first * cs, n * cs, nullptr));
                dev(vsag_amd_memcpy_h2d(dlabels.p, bucket_of.data() + first, n * 4, nullptr));
                if (with_bias) {
                    dbias.reserve(n * 4);
                    dev(vsag_amd_memcpy_h2d(dbias.p, bias.data() + first, n * 4, nullptr));
                }
                dev(vsag_amd_store_append_lists(lists.s, dcodes.as<uint8_t>(), dlabels.as<int32_t>(),
                                                with_bias ? dbias.as<float>() : nullptr, n, nullptr));
            }
            dev(vsag_amd_store_expect_stored_codes(lists.s, 0));
        }

        // label_table
        r.seek(static_cast<uint64_t>(offsets["label_table"].GetInt()));
        std::vector<int64_t> labels;
        r.vec(labels);
        if (labels.size() < total) {
            throw VsagException(ErrorType::INVALID_BINARY, "the serialized label table is shorter than the index");
        }
        labels.resize(total);

        // reorder_codes
        Quantizer pq = pq_.blank();
        StoreHandle precise;
        DevBuf raw;
        if (use_reorder_) {
            CHECK_ARGUMENT(offsets.Contains("reorder_codes"),
                           "the serialized index keeps its precise codes list by list (precise_codes_layout = bucket), "
                           "which is not read here");
            r.seek(static_cast<uint64_t>(offsets["reorder_codes"].GetInt()));
            const uint64_t n = pq_.kind == VSAG_AMD_KIND_FP32 ? read_flat_cell(r, pq, nullptr, &raw)
                                                              : read_flat_cell(r, pq, &precise, nullptr);
            if (n != total) {
                throw VsagException(ErrorType::INVALID_BINARY, "the serialized precise codes do not cover the index");
            }
        }
        dev(vsag_amd_stream_synchronize(nullptr));

        q_.take(q);
        pq_.take(pq);
        std::swap(lists_.s, lists.s);
        std::swap(centroid_store_.s, router.s);
        std::swap(precise_.s, precise.s);
        std::swap(centroids_.p, centroids_dev.p);
        std::swap(centroids_.bytes, centroids_dev.bytes);
        std::swap(raw_.p, raw.p);
        std::swap(raw_.bytes, raw.bytes);
        labels_.swap(labels);
        rebuild_label_map(labels_, known_);
        trained_ = file_trained;
    }

    // The router of the reference is an hgraph over the centroids (ivf_nearest_partition.cpp:150-153); of its image
    // (hgraph_serialize.cpp:286-311,397-401) the label table and the flat cell of fp32 codes that follows it are read:
    // centroid b is the code whose label is b.
    void
    read_router_image(Reader& r, std::vector<float>& centroids) const {
        std::vector<int64_t> labels;
        r.vec(labels);
        r.skip(r.get<uint64_t>() * 12);  // the label -> inner id pairs
        if (r.length() - r.cursor() >= 8) {
            if (r.get<uint64_t>() == 0x534F555243454944ULL) {  // a table of source ids
                const auto count = r.get<uint64_t>();
                for (uint64_t i = 0; i < count; ++i) {
                    r.skip(r.get<uint64_t>());
                }
            } else {
                r.seek(r.cursor() - 8);
            }
        }
        const auto total = r.get<uint32_t>();
        (void)r.get<uint32_t>();
        const auto cs = r.get<uint32_t>();
        const auto bytes = r.get<uint64_t>();
        if (cs != 4 * q_.dim || total != labels.size() || total != nlist_ || bytes < static_cast<uint64_t>(total) * cs) {
            throw VsagException(ErrorType::INVALID_BINARY, "the router image does not hold one fp32 centroid per bucket");
        }
        std::vector<float> rows(static_cast<size_t>(total) * q_.dim);
        r.read(rows.data(), rows.size() * 4);
        centroids.assign(rows.size(), 0.0F);
        for (uint32_t i = 0; i < total; ++i) {
            if (labels[i] < 0 || labels[i] >= static_cast<int64_t>(nlist_)) {
                throw VsagException(ErrorType::INVALID_BINARY, "the router image names a bucket that does not exist");
            }
            std::memcpy(centroids.data() + static_cast<size_t>(labels[i]) * q_.dim, rows.data() + static_cast<size_t>(i) * q_.dim,
                        static_cast<size_t>(q_.dim) * 4);
        }
    }

private:
    void
    check_usable() const {
        if (broken_) {
            throw VsagException(ErrorType::INTERNAL_ERROR, "an insert failed part-way on the device: the index is unusable");
        }
    }

    static void
    fetch(SearchContext& ctx, const DevBuf& ids_dev, const DevBuf& d_dev, size_t count, std::vector<uint32_t>& ids,
          std::vector<float>& dists) {
        ids.resize(count);
        dists.resize(count);
        ctx.download_later(ids.data(), ids_dev.p, count * 4);
        ctx.download(dists.data(), d_dev.p, count * 4);
    }

    // Codes in the lists of ctx.buckets, over all (query, list) pairs.
    uint64_t
    probed_codes(SearchContext& ctx, int64_t nq, uint32_t nprobe) const {
        ctx.scalar.reserve(8);
        dev(vsag_amd_ivf_probed_codes(lists_.s, ctx.buckets.as<int32_t>(), nq, nprobe, ctx.scalar.as<uint64_t>(),
                                      ctx.stream));
        uint64_t total = 0;
        ctx.download(&total, ctx.scalar.p, 8);
        return total;
    }

    // Scan of the lists in ctx.buckets for the uploaded queries: kc (distance, posting id) per query, ascending, in
    // ctx.cand_ids / ctx.cand_d.
    void
    scan_lists(SearchContext& ctx, int64_t nq, uint32_t nprobe, uint32_t kc, const vsag_amd_search_options_t& opt) const {
        ctx.cand_ids.reserve(static_cast<size_t>(nq) * kc * 4);
        ctx.cand_d.reserve(static_cast<size_t>(nq) * kc * 4);
        const size_t wsb = vsag_amd_ivf_scan_workspace_bytes(lists_.s, nq, nprobe, kc);
        ctx.workspace.reserve(wsb);
        dev(vsag_amd_ivf_scan_topk_ex(lists_.s, ctx.queries.as<float>(), nq, ctx.buckets.as<int32_t>(), nprobe, kc, &opt,
                                      ctx.cand_ids.as<uint32_t>(), ctx.cand_d.as<float>(), ctx.workspace.p, wsb,
                                      ctx.stream));
    }

    // Posting ids to vectors (ivf.cpp:1799-1826): per query the smallest distance of every vector, ascending, the best
    // `keep` kept.  The rows shrink from kc to keep entries.
    void
    merge_postings(std::vector<uint32_t>& ids, std::vector<float>& dists, int64_t nq, uint32_t kc, uint32_t keep) const {
        std::vector<uint32_t> out_ids(static_cast<size_t>(nq) * keep, VSAG_AMD_INVALID_ID);
        std::vector<float> out_d(out_ids.size(), std::numeric_limits<float>::infinity());
        std::unordered_set<uint32_t> seen;
        for (int64_t q = 0; q < nq; ++q) {
            seen.clear();
            uint32_t w = 0;
            for (uint32_t i = 0; i < kc && w < keep; ++i) {
                const uint32_t id = ids[q * kc + i];
                if (id == VSAG_AMD_INVALID_ID) {
                    break;
                }
                if (seen.insert(id / bpd_).second) {
                    out_ids[q * keep + w] = id / bpd_;
                    out_d[q * keep + w] = dists[q * kc + i];
                    ++w;
                }
            }
        }
        ids.swap(out_ids);
        dists.swap(out_d);
    }

    // FlattenReorder::Reorder (impl/reorder/flatten_reorder.cpp:52-114): distances of the candidates (nq x kcand inner
    // ids, VSAG_AMD_INVALID_ID = none) by the precise codes, the best `keep` per query, ascending.  Returns the number
    // of distances evaluated.
    uint64_t
    rerank(SearchContext& ctx, int64_t nq, const std::vector<uint32_t>& cand, uint32_t kcand, uint32_t keep,
           std::vector<uint32_t>& ids, std::vector<float>& dists) const {
        uint64_t evaluated = 0;
        for (uint32_t id : cand) {
            evaluated += id != VSAG_AMD_INVALID_ID ? 1 : 0;
        }
        ctx.upload(ctx.cand_ids, cand.data(), cand.size() * 4);
        if (pq_.kind == VSAG_AMD_KIND_FP32) {
            ctx.out_ids.reserve(static_cast<size_t>(nq) * keep * 4);
            ctx.out_d.reserve(static_cast<size_t>(nq) * keep * 4);
            dev(vsag_amd_rerank_fp32(raw_.as<float>(), labels_.size(), q_.dim, q_.metric, ctx.queries.as<float>(), nq,
                                     ctx.cand_ids.as<uint32_t>(), kcand, keep, ctx.out_ids.as<uint32_t>(),
                                     ctx.out_d.as<float>(), ctx.stream));
            fetch(ctx, ctx.out_ids, ctx.out_d, static_cast<size_t>(nq) * keep, ids, dists);
            return evaluated;
        }
        ctx.out_d.reserve(static_cast<size_t>(nq) * kcand * 4);
        const size_t wsb = vsag_amd_store_distances_workspace_bytes(precise_.s, nq);
        ctx.workspace.reserve(wsb);
        dev(vsag_amd_store_distances(precise_.s, ctx.queries.as<float>(), nq, ctx.cand_ids.as<uint32_t>(), kcand,
                                     ctx.out_d.as<float>(), ctx.workspace.p, wsb, ctx.stream));
        std::vector<float> exact(static_cast<size_t>(nq) * kcand);
        ctx.download(exact.data(), ctx.out_d.p, exact.size() * 4);
        ids.assign(static_cast<size_t>(nq) * keep, VSAG_AMD_INVALID_ID);
        dists.assign(ids.size(), std::numeric_limits<float>::infinity());
        std::vector<std::pair<float, uint32_t>> row;
        for (int64_t q = 0; q < nq; ++q) {
            row.clear();
            for (uint32_t i = 0; i < kcand; ++i) {
                if (cand[q * kcand + i] != VSAG_AMD_INVALID_ID) {
                    row.emplace_back(exact[q * kcand + i], cand[q * kcand + i]);
                }
            }
            std::sort(row.begin(), row.end());
            for (uint32_t i = 0; i < keep && i < row.size(); ++i) {
                dists[q * keep + i] = row[i].first;
                ids[q * keep + i] = row[i].second;
            }
        }
        return evaluated;
    }

    // The nearest `per_row` centroids of n rows under the index metric (IVFNearestPartition::ClassifyDatas,
    // ivf_nearest_partition.cpp:88-147, exact instead of through the router graph): n x per_row list numbers.
    void
    classify(const float* x_dev, uint64_t n, uint32_t per_row, DevBuf& buckets) const {
        classify_with(centroid_store_.s, x_dev, n, per_row, buckets);
    }
    void
    classify_with(const vsag_amd_store_t* router, const float* x_dev, uint64_t n, uint32_t per_row, DevBuf& buckets) const {
        buckets.reserve(std::max<size_t>(n * per_row * 4, 4));
        DevBuf d, ws;
        const uint64_t chunk = 65536;
        d.reserve(std::min(n, chunk) * per_row * 4);
        for (uint64_t r0 = 0; r0 < n; r0 += chunk) {
            const uint64_t nr = std::min(chunk, n - r0);
            const size_t wsb = vsag_amd_ivf_route_workspace_bytes(router, nr, per_row);
            ws.reserve(wsb);
            dev(vsag_amd_ivf_route(router, x_dev + r0 * q_.dim, nr, per_row,
                                   buckets.as<int32_t>() + r0 * per_row, d.as<float>(), ws.p, wsb, nullptr));
        }
        dev(vsag_amd_stream_synchronize(nullptr));
    }

    // IVF::Train (ivf.cpp:564-588): sample, k-means (25 iterations, hard-coded in ivf_nearest_partition.cpp:65-70),
    // quantizer training on the same sample (on its residuals with use_residual, bucket_datacell.h:594-619); the
    // precise quantizer is trained on all of the data.  x_all_dev: the rows on the device when the caller has them.
    void
    train_locked(const DatasetPtr& base, const std::vector<int64_t>& rows, const float* x_all_dev) {
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
        // "random": the centroids are nlist rows of the shuffled sample.  "kmeans": k-means++ seeding, the default
        // of KMeansCluster::Run (kmeans_cluster.cpp:78-82, 383-435), with draws from the seeded generator where the
        // reference seeds an mt19937 from std::random_device; then the Lloyd iterations.
        DevBuf centroids;
        centroids.reserve(static_cast<size_t>(nlist_) * q_.dim * 4);
        dev(vsag_amd_memcpy_d2d(centroids.p, sample_dev.p, static_cast<size_t>(nlist_) * q_.dim * 4, nullptr));
        if (!train_random_) {
            {
                std::uniform_int_distribution<uint64_t> first_dis(0, sample_n - 1);
                const uint64_t first = first_dis(gen);
                std::uniform_real_distribution<double> unit(0.0, 1.0);
                std::vector<double> draws(nlist_ > 1 ? nlist_ - 1 : 0);
                for (double& d : draws) {
                    d = unit(gen);
                    d = d < 1.0 ? d : 0.0;
                }
                DevBuf ws;
                size_t wsb = vsag_amd_kmeans_init_plus_plus_workspace_bytes(sample_n);
                ws.reserve(wsb);
                dev(vsag_amd_kmeans_init_plus_plus(sample_dev.as<float>(), sample_n, q_.dim, nlist_, first, draws.data(),
                                                   centroids.as<float>(), nullptr, ws.p, wsb, nullptr));
                dev(vsag_amd_stream_synchronize(nullptr));
            }
            DevBuf labels, ws;
            labels.reserve(sample_n * 4);
            size_t wsb = vsag_amd_kmeans_run_workspace_bytes(sample_n, q_.dim, nlist_);
            ws.reserve(wsb);
            double loss = 0;
            dev(vsag_amd_kmeans_run(sample_dev.as<float>(), sample_n, q_.dim, centroids.as<float>(), nlist_, 25, 47,
                                    labels.as<int32_t>(), &loss, ws.p, wsb, nullptr));
        }
        if (q_.metric == VSAG_AMD_METRIC_COSINE) {
            // the router keeps unit centroids (ivf_nearest_partition.cpp:81-85), and so do the residuals
            std::vector<float> c(static_cast<size_t>(nlist_) * q_.dim);
            dev(vsag_amd_memcpy_d2h(c.data(), centroids.p, c.size() * 4, nullptr));
            for (uint32_t l = 0; l < nlist_; ++l) {
                float* row = c.data() + static_cast<size_t>(l) * q_.dim;
                float s = 0.0F;
                for (uint32_t d = 0; d < q_.dim; ++d) {
                    s += row[d] * row[d];
                }
                const float norm = std::sqrt(s);
                for (uint32_t d = 0; d < q_.dim && norm > 0.0F; ++d) {
                    row[d] /= norm;
                }
            }
            dev(vsag_amd_memcpy_h2d(centroids.p, c.data(), c.size() * 4, nullptr));
        }
        // Router: an fp32 store of the centroids under the index metric.
        Quantizer cq;
        cq.kind = VSAG_AMD_KIND_FP32;
        cq.metric = q_.metric;
        cq.dim = q_.dim;
        StoreHandle router;
        router.s = cq.make_store();
        dev(vsag_amd_store_append(router.s, centroids.as<uint8_t>(), nlist_, nullptr));
        dev(vsag_amd_stream_synchronize(nullptr));
        // Router, quantizers, lists and precise store are built beside what the index holds and change hands together
        // at the end: a step that throws leaves the index as it was.
        Quantizer q = q_.blank();
        if (use_residual_) {
            DevBuf nearest, residuals;
            classify_with(router.s, sample_dev.as<float>(), sample_n, 1, nearest);
            residuals.reserve(sample.size() * 4);
            dev(vsag_amd_residual_rows(sample_dev.as<float>(), sample_n, q_.dim, q_.metric, nearest.as<int32_t>(),
                                       centroids.as<float>(), residuals.as<float>(), nullptr));
            q.train(residuals.as<float>(), sample_n);
        } else {
            q.train(sample_dev.as<float>(), sample_n);
        }
        StoreHandle lists;
        lists.s = q.make_store();
        if (use_residual_) {
            dev(vsag_amd_store_set_residual(lists.s, centroids.as<float>(), nlist_, nullptr));
        }
        dev(vsag_amd_store_set_lists(lists.s, nullptr, nullptr, 0, nlist_, nullptr));
        Quantizer pq = pq_.blank();
        StoreHandle precise;
        const bool precise_codes = use_reorder_ && pq_.kind != VSAG_AMD_KIND_FP32;
        if (precise_codes) {
            DevBuf x;
            if (x_all_dev == nullptr) {
                upload_rows(base, rows, q_.dim, x);
                x_all_dev = x.as<float>();
            }
            pq.train(x_all_dev, n);
            precise.s = pq.make_store();
        }
        dev(vsag_amd_stream_synchronize(nullptr));
        q_.take(q);
        if (precise_codes) {
            pq_.take(pq);
            std::swap(precise_.s, precise.s);
        }
        std::swap(centroid_store_.s, router.s);
        std::swap(centroids_.p, centroids.p);
        std::swap(centroids_.bytes, centroids.bytes);
        std::swap(lists_.s, lists.s);
        trained_ = true;
    }

    // IVF::Add (ivf.cpp:590-724).
    std::vector<int64_t>
    add_locked(const DatasetPtr& base, bool train_first) {
        check_usable();
        check_base(base, q_.dim);
        if (!train_first && !trained_) {
            throw VsagException(ErrorType::INTERNAL_ERROR, "ivf index add without train error");
        }
        std::vector<int64_t> rows;
        std::vector<int64_t> failed = split_new_rows(base, known_, rows);
        if (rows.empty()) {
            return failed;
        }
        const uint64_t n_new = rows.size();
        const uint64_t n_old = labels_.size();
        CHECK_ARGUMENT((n_old + n_new) * bpd_ < VSAG_AMD_INVALID_ID, "the lists hold at most 2^32 - 2 postings");
        DevBuf x;
        upload_rows(base, rows, q_.dim, x);
        if (!trained_) {
            train_locked(base, rows, x.as<float>());
        }
        // the lists of every row, nearest first; posting (i, j) is row i in list buckets[i * bpd + j]
        DevBuf buckets;
        classify(x.as<float>(), n_new, bpd_, buckets);
        const uint64_t postings = n_new * bpd_;
        DevBuf expanded;
        const float* xe = x.as<float>();
        if (bpd_ > 1) {
            upload_rows(base, rows, q_.dim, expanded, bpd_);
            xe = expanded.as<float>();
        }
        DevBuf residuals, codes, bias;
        if (use_residual_) {
            residuals.reserve(postings * q_.dim * 4);
            dev(vsag_amd_residual_rows(xe, postings, q_.dim, q_.metric, buckets.as<int32_t>(), centroids_.as<float>(),
                                       residuals.as<float>(), nullptr));
            xe = residuals.as<float>();
        }
        const uint8_t* code_src = reinterpret_cast<const uint8_t*>(xe);
        if (q_.kind != VSAG_AMD_KIND_FP32) {
            codes.reserve(postings * q_.code_size());
            q_.encode(xe, postings, codes.as<uint8_t>());
            code_src = codes.as<uint8_t>();
        }
        const float* bias_src = nullptr;
        if (use_residual_ && q_.metric == VSAG_AMD_METRIC_L2) {
            DevBuf decoded;
            bias.reserve(postings * 4);
            decoded.reserve(postings * q_.dim * 4);
            dev(vsag_amd_residual_bias(lists_.s, code_src, postings, buckets.as<int32_t>(), centroids_.as<float>(),
                                       bias.as<float>(), decoded.as<float>(), nullptr));
            dev(vsag_amd_stream_synchronize(nullptr));
            bias_src = bias.as<float>();
        }
        // From here on two structures change; a failure between them leaves them out of step.
        try {
            if (use_reorder_ && pq_.kind == VSAG_AMD_KIND_FP32) {
                const size_t row_bytes = static_cast<size_t>(q_.dim) * 4;
                raw_.grow((n_old + n_new) * row_bytes, n_old * row_bytes);
                dev(vsag_amd_memcpy_d2d(raw_.as<uint8_t>() + n_old * row_bytes, x.p, n_new * row_bytes, nullptr));
            } else if (use_reorder_) {
                DevBuf pcodes;
                pcodes.reserve(n_new * pq_.code_size());
                pq_.encode(x.as<float>(), n_new, pcodes.as<uint8_t>());
                dev(vsag_amd_store_append(precise_.s, pcodes.as<uint8_t>(), n_new, nullptr));
                dev(vsag_amd_stream_synchronize(nullptr));
            }
            dev(vsag_amd_store_append_lists(lists_.s, code_src, buckets.as<int32_t>(), bias_src, postings, nullptr));
            dev(vsag_amd_stream_synchronize(nullptr));
        } catch (...) {
            broken_ = n_old > 0 || vsag_amd_store_size(lists_.s) != 0;
            throw;
        }
        for (int64_t r : rows) {
            known_.emplace(base->GetIds()[r], static_cast<uint32_t>(labels_.size()));
            labels_.push_back(base->GetIds()[r]);
        }
        return failed;
    }

    CommonParam common_;
    Quantizer q_;   // codes of the lists
    Quantizer pq_;  // precise codes of the rerank (fp32: the raw rows)
    uint32_t nlist_ = 10;
    uint32_t bpd_ = 1;  // buckets_per_data
    bool use_reorder_ = false;
    bool use_residual_ = false;
    bool train_random_ = false;
    int64_t train_sample_count_ = 65536;
    bool trained_ = false;
    bool broken_ = false;
    StoreHandle centroid_store_, lists_, precise_;
    DevBuf centroids_, raw_;
    std::vector<int64_t> labels_;
    LabelMap known_;
};

}  // namespace

Expected<std::shared_ptr<Index>>
Factory::CreateIndex(const std::string& name, const std::string& parameters, Allocator* allocator) {
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
        std::shared_ptr<GpuIndex> index;
        if (name == "brute_force") {
            index = std::make_shared<BruteForce>(common, index_param);
        } else if (name == "ivf") {
            index = std::make_shared<IVF>(common, index_param);
        }
        if (index != nullptr) {
            index->set_allocator(allocator);
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

}  // namespace amd_gpu
}  // namespace vsag
