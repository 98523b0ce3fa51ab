// Error plumbing and the entry points that are not tied to one layer.
#include "common.hpp"

#include <cstring>
#include <mutex>
#include <string>
#include <vector>

namespace cnt {
namespace {
thread_local char g_error[512] = "";
}

void set_error(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}
const char *last_error() { return g_error; }
}  // namespace cnt

namespace cnt {
namespace {
struct ProfRecord {
    std::string label;
    hipEvent_t start, stop;
};
std::mutex g_prof_mutex;
bool g_prof_on = false;
std::vector<ProfRecord> g_prof_records;
std::vector<hipEvent_t> g_prof_pool;

hipEvent_t prof_event() {
    if (!g_prof_pool.empty()) {
        hipEvent_t e = g_prof_pool.back();
        g_prof_pool.pop_back();
        return e;
    }
    hipEvent_t e = nullptr;
    if (hipEventCreate(&e) != hipSuccess) return nullptr;
    return e;
}
}  // namespace

ProfileScope::ProfileScope(hipStream_t stream, const char *label) : stream_(stream), slot_(-1) {
    if (!g_prof_on || !label) return;
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    ProfRecord r;
    r.label = label;
    r.start = prof_event();
    r.stop = prof_event();
    if (!r.start || !r.stop) return;
    (void)hipEventRecord(r.start, stream);
    g_prof_records.push_back(r);
    slot_ = (int)g_prof_records.size() - 1;
}
ProfileScope::~ProfileScope() {
    if (slot_ < 0) return;
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    if (slot_ < (int)g_prof_records.size()) (void)hipEventRecord(g_prof_records[slot_].stop, stream_);
}
}  // namespace cnt

extern "C" {

int cnt_profile_enable(int on) {
    std::lock_guard<std::mutex> lock(cnt::g_prof_mutex);
    for (auto &r : cnt::g_prof_records) {
        cnt::g_prof_pool.push_back(r.start);
        cnt::g_prof_pool.push_back(r.stop);
    }
    cnt::g_prof_records.clear();
    cnt::g_prof_on = (on != 0);
    return CNT_OK;
}

int cnt_profile_get(int index, char *label, int label_cap, int *launches, float *total_ms) {
    using namespace cnt;
    std::lock_guard<std::mutex> lock(g_prof_mutex);
    // distinct labels in order of first appearance
    std::vector<std::string> labels;
    for (auto &r : g_prof_records) {
        bool seen = false;
        for (auto &l : labels) seen = seen || (l == r.label);
        if (!seen) labels.push_back(r.label);
    }
    if (index < 0 || index >= (int)labels.size()) return CNT_ERR_ARG;
    int n = 0;
    float total = 0.0f;
    for (auto &r : g_prof_records) {
        if (r.label != labels[index]) continue;
        CNT_HIP(hipEventSynchronize(r.stop));
        float ms = 0.0f;
        CNT_HIP(hipEventElapsedTime(&ms, r.start, r.stop));
        total += ms;
        ++n;
    }
    if (label && label_cap > 0) {
        std::strncpy(label, labels[index].c_str(), (size_t)label_cap - 1);
        label[label_cap - 1] = 0;
    }
    if (launches) *launches = n;
    if (total_ms) *total_ms = total;
    return CNT_OK;
}

int cnt_version(void) { return 1; }
const char *cnt_last_error(void) { return cnt::last_error(); }

int cnt_matrix_product(void *stream, float *C, int m, int n, int k, const float *A, int transA, const float *B,
                       int transB, int accumulate) {
    using namespace cnt;
    CNT_REQUIRE(C && A && B, "matrix_product: null argument");
    // helpers/Matrix.cu has no functor for this combination either
    CNT_REQUIRE(!(transA && transB), "matrix_product: transposing both operands is not supported");
    return gemm_simple(static_cast<hipStream_t>(stream), C, m, n, k, A, transA != 0, B, transB != 0,
                       accumulate != 0);
}

}  // extern "C"
