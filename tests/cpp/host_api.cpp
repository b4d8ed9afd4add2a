// A C++ consumer of the host layer, written the way a program uses the reference's public API
// (examples/cpp/101_index_hnsw.cpp style: Factory::CreateIndex -> Build -> KnnSearch; include/vsag/factory.h:47-50 with
// its Allocator argument, include/vsag/index.h, include/vsag/dataset.h:140-147).  Prints one line per check and
// returns the number of failed checks; with no GPU the factory's error is the expected outcome (exit code 100).
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <sstream>
#include <string>
#include <vector>

#include "vsag_host.h"

namespace {

// Counts what goes through it, like the allocators the reference's tests hand to the factory.
class CountingAllocator : public vsag::Allocator {
public:
    std::string
    Name() override {
        return "counting";
    }
    void*
    Allocate(uint64_t size) override {
        void* p = std::malloc(size);
        live_[p] = size;
        ++allocations_;
        return p;
    }
    void
    Deallocate(void* p) override {
        if (p == nullptr) {
            return;
        }
        if (live_.erase(p) == 0) {
            ++foreign_frees_;
        }
        std::free(p);
    }
    void*
    Reallocate(void* p, uint64_t size) override {
        void* q = std::realloc(p, size);
        live_.erase(p);
        live_[q] = size;
        return q;
    }
    std::map<void*, uint64_t> live_;
    int64_t allocations_ = 0;
    int64_t foreign_frees_ = 0;
};

int failures = 0;

void
check(bool ok, const char* what) {
    std::printf("%s %s\n", ok ? "ok  " : "FAIL", what);
    failures += ok ? 0 : 1;
}

}  // namespace

int
main() {
    const int64_t n = 5000, dim = 32, nq = 7, k = 5;
    std::mt19937 gen(11);
    std::uniform_real_distribution<float> unit(0.0F, 1.0F);
    std::vector<float> x(n * dim), q(nq * dim);
    std::vector<int64_t> ids(n);
    for (auto& v : x) {
        v = unit(gen);
    }
    for (int64_t i = 0; i < n; ++i) {
        ids[i] = 1000 + i;
    }
    for (int64_t i = 0; i < nq; ++i) {
        for (int64_t d = 0; d < dim; ++d) {
            q[i * dim + d] = x[(17 * i + 3) * dim + d];  // stored rows: the nearest neighbour is known
        }
    }
    const std::string params = R"({"dtype":"float32","metric_type":"l2","dim":32,"index_param":{"base_quantization_type":"fp32"}})";
    CountingAllocator allocator;
    auto created = vsag::Factory::CreateIndex("brute_force", params, &allocator);
    if (!created.has_value()) {
        std::printf("factory: %s\n", created.error().message.c_str());
        return 100;
    }
    {
        auto index = created.value();
        auto base = vsag::Dataset::Make();
        base->NumElements(n)->Dim(dim)->Ids(ids.data())->Float32Vectors(x.data())->Owner(false);
        auto built = index->Build(base);
        check(built.has_value() && built.value().empty(), "Build inserts every row");
        check(index->GetNumElements() == n, "GetNumElements");
        check(allocator.allocations_ == 0, "building takes nothing from the result allocator");

        auto query = vsag::Dataset::Make();
        query->NumElements(1)->Dim(dim)->Float32Vectors(q.data())->Owner(false);
        {
            auto result = index->KnnSearch(query, k, "{}");
            check(result.has_value(), "KnnSearch");
            if (result.has_value()) {
                auto r = result.value();
                check(r->GetDim() == k && r->GetIds()[0] == 1000 + 3 && r->GetDistances()[0] == 0.0F,
                      "the stored row is its own nearest neighbour at distance 0");
                check(allocator.live_.count(const_cast<int64_t*>(r->GetIds())) == 1 &&
                          allocator.live_.count(const_cast<float*>(r->GetDistances())) == 1,
                      "ids and distances of a result come from the allocator");
            }
        }
        check(allocator.live_.empty() && allocator.foreign_frees_ == 0, "a result gives its arrays back to the allocator");

        auto batch = vsag::Dataset::Make();
        batch->NumElements(nq)->Dim(dim)->Float32Vectors(q.data())->Owner(false);
        {
            auto result = index->KnnSearch(batch, k, "{}");
            bool good = result.has_value() && result.value()->GetNumElements() == nq && result.value()->GetDim() == k;
            for (int64_t i = 0; good && i < nq; ++i) {
                good = result.value()->GetIds()[i * k] == 1000 + 17 * i + 3;
            }
            check(good, "a batch of queries returns one row per query");
            auto dist = index->CalDistanceById(q.data(), ids.data(), 4, true, -1);
            check(dist.has_value() && dist.value()->GetDim() == 4 &&
                      allocator.live_.count(const_cast<float*>(dist.value()->GetDistances())) == 1,
                  "CalDistanceById answers through the allocator too");
        }
        check(allocator.live_.empty(), "nothing of the allocator's is left behind");

        // Serialize -> Deserialize into a second index (include/vsag/index.h:903-940)
        std::stringstream stream;
        auto saved = index->Serialize(stream);
        check(saved.has_value(), "Serialize");
        auto second = vsag::Factory::CreateIndex("brute_force", params).value();
        auto loaded = second->Deserialize(stream);
        check(loaded.has_value() && second->GetNumElements() == n, "Deserialize");
        auto again = second->KnnSearch(query, k, "{}");
        check(again.has_value() && again.value()->GetIds()[0] == 1000 + 3, "the loaded index answers like the saved one");

        auto twice = index->Build(base);
        check(!twice.has_value() && twice.error().type == vsag::ErrorType::BUILD_TWICE, "BUILD_TWICE");
        auto bad = vsag::Factory::CreateIndex("brute_force", R"({"dtype":"float32","metric_type":"l2","dim":32,"index_param":{"nonsense":1}})");
        check(!bad.has_value() && bad.error().type == vsag::ErrorType::INVALID_ARGUMENT, "unknown index_param key");
    }
    std::printf("%s\n", failures == 0 ? "all checks passed" : "some checks FAILED");
    return failures;
}
