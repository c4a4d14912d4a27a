// Error reporting, version and the host-side interval lookup table of the C ABI.
#include "kmi_common.h"
#include <algorithm>
#include <vector>
#include <new>

static thread_local char g_err[512] = "";

int kmi_set_error(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

extern "C" const char* kmi_get_last_error_string(void) { return g_err; }
extern "C" int kmi_version(void) { return 100; }

// Interval table.  Segment i covers (edge[i-1], edge[i]]; queries beyond the last edge fall into the
// last segment.  Same observable behaviour as the reference class for every m >= 1
// (kernels/csrc/kairos_kernel/lut/lut.h:22-38), with edges kept inclusive and a lower_bound search.
namespace {
struct Lut {
    std::vector<int> edge;
    std::vector<int> comp;
    int memo_m = -1;
    int memo_c = 0;
};
}  // namespace

extern "C" void* kmi_lut_new(void) {
    Lut* l = new (std::nothrow) Lut();
    if (l) {
        l->edge.reserve(32);
        l->comp.reserve(32);
    }
    return l;
}
extern "C" void kmi_lut_free(void* p) { delete static_cast<Lut*>(p); }

extern "C" int kmi_lut_record(void* p, int right_edge, int comp_type) {
    if (!p) return kmi_set_error(KMI_E_HANDLE, "kmi_lut_record: NULL table");
    Lut* l = static_cast<Lut*>(p);
    l->edge.push_back(right_edge);
    l->comp.push_back(comp_type);
    l->memo_m = -1;
    return KMI_OK;
}

extern "C" int kmi_lut_get(void* p, int m) {
    Lut* l = static_cast<Lut*>(p);
    if (!l || l->comp.empty()) return kmi_set_error(KMI_E_HANDLE, "kmi_lut_get: NULL or empty table");
    if (m == l->memo_m) return l->memo_c;
    auto it = std::lower_bound(l->edge.begin(), l->edge.end(), m);   // first edge >= m
    size_t i = (it == l->edge.end()) ? l->edge.size() - 1 : static_cast<size_t>(it - l->edge.begin());
    l->memo_m = m;
    l->memo_c = l->comp[i];
    return l->memo_c;
}

extern "C" int kmi_lut_shrink_to_fit(void* p) {
    if (!p) return kmi_set_error(KMI_E_HANDLE, "kmi_lut_shrink_to_fit: NULL table");
    Lut* l = static_cast<Lut*>(p);
    l->edge.shrink_to_fit();
    l->comp.shrink_to_fit();
    return KMI_OK;
}
extern "C" int kmi_lut_size(void* p) {
    if (!p) return kmi_set_error(KMI_E_HANDLE, "kmi_lut_size: NULL table");
    return static_cast<int>(static_cast<Lut*>(p)->comp.size());
}

// Bounded conversion buffer, host-side bookkeeping only.  The caller owns ONE device buffer of `capacity` bytes (sized
// for the largest converted weight of its model) and asks, before a lane that needs a converted copy, whether the
// buffer already holds that copy.  A request larger than the buffer is refused: the bound is the buffer, whatever
// the layers ask for.  One handle per stream of execution (requests are not ordered between streams here).
namespace {
struct ConvCache {
    void* buffer;
    size_t capacity;
    bool valid = false;
    uint64_t owner = 0;
    int format = 0;
    size_t held = 0;
    size_t high_water = 0;
    uint64_t hits = 0, misses = 0;
};
}  // namespace

extern "C" void* kmi_cache_create(void* device_buffer, size_t capacity_bytes) {
    if (!device_buffer || capacity_bytes == 0 || !kmi_aligned16(device_buffer)) {
        kmi_set_error(device_buffer && !kmi_aligned16(device_buffer) ? KMI_E_ALIGN : KMI_E_NULL,
                      "kmi_cache_create: needs a 16-byte aligned device buffer and a capacity");
        return nullptr;
    }
    ConvCache* c = new (std::nothrow) ConvCache();
    if (c) {
        c->buffer = device_buffer;
        c->capacity = capacity_bytes;
    }
    return c;
}
extern "C" void kmi_cache_destroy(void* p) { delete static_cast<ConvCache*>(p); }

extern "C" int kmi_cache_acquire(void* p, uint64_t owner, int format, size_t nbytes, void** out_ptr) {
    ConvCache* c = static_cast<ConvCache*>(p);
    if (!c) return kmi_set_error(KMI_E_HANDLE, "kmi_cache_acquire: NULL cache");
    if (!out_ptr) return kmi_set_error(KMI_E_NULL, "kmi_cache_acquire: out_ptr is NULL");
    if (nbytes == 0 || nbytes > c->capacity)
        return kmi_set_error(KMI_E_SHAPE, "kmi_cache_acquire: %zu bytes asked of a buffer of %zu", nbytes, c->capacity);
    *out_ptr = c->buffer;
    if (nbytes > c->high_water) c->high_water = nbytes;
    const bool hit = c->valid && c->owner == owner && c->format == format && c->held == nbytes;
    c->valid = true;
    c->owner = owner;
    c->format = format;
    c->held = nbytes;
    if (hit) ++c->hits; else ++c->misses;
    return hit ? 1 : 0;
}

extern "C" int kmi_cache_invalidate(void* p) {
    if (!p) return kmi_set_error(KMI_E_HANDLE, "kmi_cache_invalidate: NULL cache");
    static_cast<ConvCache*>(p)->valid = false;
    return KMI_OK;
}

extern "C" int kmi_cache_stats(void* p, size_t* capacity, size_t* high_water, uint64_t* hits, uint64_t* misses) {
    ConvCache* c = static_cast<ConvCache*>(p);
    if (!c) return kmi_set_error(KMI_E_HANDLE, "kmi_cache_stats: NULL cache");
    if (capacity) *capacity = c->capacity;
    if (high_water) *high_water = c->high_water;
    if (hits) *hits = c->hits;
    if (misses) *misses = c->misses;
    return KMI_OK;
}
