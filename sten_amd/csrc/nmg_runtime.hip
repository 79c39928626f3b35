// Library runtime: error state, pattern-order tables on host and device.
#include "nmg_common.h"

#include <cstdarg>
#include <algorithm>
#include <cstdio>
#include <map>
#include <mutex>
#include <vector>

namespace nmg {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

int hip_fail(hipError_t e, const char *what, const char *file, int line)
{
    set_error("HIP error %s (%s) at %s:%d in %s", hipGetErrorName(e), hipGetErrorString(e), file,
              line, what);
    return NMG_ERR_HIP;
}

int64_t binom(int m, int n)
{
    if (n < 0 || n > m) return 0;
    int64_t r = 1;
    for (int i = 1; i <= n; i++) r = r * (m - n + i) / i;
    return r;
}

// Pattern order: all increasing n-tuples of range(m), neighbours differing in one slot.
// Built bottom-up from the recurrence
//   T(n, m, flip) = maybe_reversed(T(n, m-1, true)) ++ [t + (m-1) for t in T(n-1, m-1, !flip)]
// with T(n, n) = T(0, m) = [range(n)]  (reference: grouped_nm_tensor.py:37-50).
using Table = std::vector<std::vector<int8_t>>;

static Table build_order(int n, int m, bool flip)
{
    if (n == m || n == 0) {
        std::vector<int8_t> t(n);
        for (int j = 0; j < n; j++) t[j] = (int8_t)j;
        return Table{t};
    }
    Table head = build_order(n, m - 1, true);
    if (flip) std::reverse(head.begin(), head.end());
    Table tail = build_order(n - 1, m - 1, !flip);
    for (auto &t : tail) {
        t.push_back((int8_t)(m - 1));
        head.push_back(t);
    }
    return head;
}

static std::mutex g_mu;
static std::map<std::pair<int, int>, std::vector<int8_t>> g_host_tables;

const int8_t *host_order(int n, int m)
{
    if (n < 0 || m < 1 || n > m || m > 64) return nullptr;
    std::lock_guard<std::mutex> lk(g_mu);
    auto key = std::make_pair(n, m);
    auto it = g_host_tables.find(key);
    if (it == g_host_tables.end()) {
        Table t = build_order(n, m, false);
        std::vector<int8_t> flat;
        flat.reserve(t.size() * (size_t)n);
        for (auto &row : t) flat.insert(flat.end(), row.begin(), row.end());
        if (flat.empty()) flat.push_back(0);
        it = g_host_tables.emplace(key, std::move(flat)).first;
    }
    return it->second.data();
}

// Device-side table: one file-scope array per GPU, addressed through hipGetSymbolAddress.
static __device__ __align__(256) int8_t g_order_dev[kOrderPoolBytes];

struct DevTables {
    int8_t *base = nullptr;
    size_t used = 0;                                   // bytes of the pool handed out
    std::map<std::pair<int, int>, size_t> offset;      // (n, m) -> offset of its table
};
static std::map<int, DevTables> g_dev_tables;

int device_order(int n, int m, const int8_t **d_order)
{
    const int8_t *h = host_order(n, m);
    NMG_REQUIRE(h != nullptr, NMG_ERR_ARG, "invalid n:m = %d:%d", n, m);
    int64_t bytes = binom(m, n) * n;
    NMG_REQUIRE(bytes <= kOrderSlotBytes, NMG_ERR_UNSUPPORTED,
                "pattern table of %d:%d needs %lld bytes, limit %d", n, m, (long long)bytes,
                kOrderSlotBytes);
    int dev = 0;
    NMG_HIP_TRY(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lk(g_mu);
    DevTables &dt = g_dev_tables[dev];
    if (dt.base == nullptr) {
        void *p = nullptr;
        NMG_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(g_order_dev)));
        dt.base = (int8_t *)p;
    }
    auto it = dt.offset.find(std::make_pair(n, m));
    if (it != dt.offset.end()) {
        *d_order = dt.base + it->second;
        return NMG_OK;
    }
    const size_t need = ((size_t)bytes + 15) & ~(size_t)15;
    NMG_REQUIRE(dt.used + need <= (size_t)kOrderPoolBytes, NMG_ERR_UNSUPPORTED,
                "pattern tables of this device are full (%d bytes): too many distinct n:m pairs",
                kOrderPoolBytes);
    int8_t *dst = dt.base + dt.used;
    if (bytes > 0) NMG_HIP_TRY(hipMemcpy(dst, h, (size_t)bytes, hipMemcpyHostToDevice));
    dt.offset.emplace(std::make_pair(n, m), dt.used);
    dt.used += need > 0 ? need : 16;
    *d_order = dst;
    return NMG_OK;
}

// 256 zero bytes per GPU: the source of DMA loads that must deliver zeros (reduction positions
// beyond the end of an operand).  File-scope device arrays start out zero and nothing writes it.
static __device__ __align__(256) unsigned char g_zero_page[256];
static std::map<int, const void *> g_zero_pages;

int device_zero_page(const void **d_zero)
{
    int dev = 0;
    NMG_HIP_TRY(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_zero_pages.find(dev);
    if (it == g_zero_pages.end()) {
        void *p = nullptr;
        NMG_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(g_zero_page)));
        it = g_zero_pages.emplace(dev, p).first;
    }
    *d_zero = it->second;
    return NMG_OK;
}

}  // namespace nmg

extern "C" {

int nmg_version(void) { return 1; }

const char *nmg_last_error(void) { return nmg::g_err; }

int64_t nmg_chunk(int n, int m) { return nmg::binom(m, n); }

int64_t nmg_order(int n, int m, int8_t *out)
{
    const int8_t *h = nmg::host_order(n, m);
    if (h == nullptr || out == nullptr) {
        nmg::set_error("nmg_order: invalid n:m = %d:%d or null output", n, m);
        return -1;
    }
    int64_t c = nmg::binom(m, n);
    for (int64_t i = 0; i < c * n; i++) out[i] = h[i];
    return c;
}

}  // extern "C"
