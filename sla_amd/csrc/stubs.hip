// Entry points whose kernels are not written yet: they fail loudly.
#include "common.h"
namespace sla {
int64_t sage_quant_workspace_bytes(int, int, int) { return 256; }
}
using namespace sla;
#define NOT_YET(name) do { set_error(name ": not implemented"); return SLA_ERR_UNSUPPORTED; } while (0)
extern "C" int sage_quant_qk(const void*, const void*, int, int, int, int, int, int, int, int8_t*, float*, int8_t*, float*, void*, int64_t, void*) { NOT_YET("sage_quant_qk"); }
extern "C" int sage_quant_v(const void*, int, int, int, int, int, uint8_t*, float*, void*, int64_t, void*) { NOT_YET("sage_quant_v"); }
extern "C" int sage_sparse_attn_fwd(const int8_t*, const float*, const int8_t*, const float*, const uint8_t*, const float*, const void*, int, void*, int, int, int, int, int, int, int, int, float, void*) { NOT_YET("sage_sparse_attn_fwd"); }
