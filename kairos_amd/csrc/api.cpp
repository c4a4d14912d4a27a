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
