// Test infrastructure only: C-callable wrapper around the REFERENCE's own LUT class
// (kernels/csrc/kairos_kernel/lut/lut.h:8-45), compiled from where it lies under the reference
// tree (include path given by the Makefile).  Nothing from the reference is copied here.
#include "lut.h"

extern "C" {
void* ref_lut_new() { return new LUT(); }
void ref_lut_free(void* p) { delete static_cast<LUT*>(p); }
void ref_lut_record(void* p, int r, int comp) { static_cast<LUT*>(p)->record(r, comp); }
int ref_lut_get(void* p, int m) { return static_cast<LUT*>(p)->get(m); }
void ref_lut_shrink_to_fit(void* p) { static_cast<LUT*>(p)->shrink_to_fit(); }
}
