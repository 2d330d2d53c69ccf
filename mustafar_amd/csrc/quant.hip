// Quantised entry points: report MSTF_EUNSUPPORTED until the quantised kernels are in place.
#include "common.hpp"
extern "C" size_t mstf_compress_quant_workspace_bytes(int, int, int) { return 0; }
extern "C" int mstf_compress_key_quant(void*, const mstf_half*, int, int, int, int, int, uint64_t*, uint32_t*, uint32_t*, uint32_t*, mstf_half*, mstf_half*, uint64_t*, uint32_t*, uint64_t, void*, size_t) { return MSTF_EUNSUPPORTED; }
extern "C" int mstf_compress_value_quant(void*, const mstf_half*, int, int, int, int, int, uint64_t*, uint32_t*, uint32_t*, uint32_t*, mstf_half*, mstf_half*, uint64_t*, uint32_t*, uint64_t, void*, size_t) { return MSTF_EUNSUPPORTED; }
extern "C" int mstf_key_spmv_quant(void*, const uint64_t*, const uint32_t*, const uint32_t*, const uint32_t*, const uint32_t*, const mstf_half*, const mstf_half*, const mstf_half*, mstf_half*, int, int, int, int, int, int, int, int) { return MSTF_EUNSUPPORTED; }
extern "C" size_t mstf_value_spmv_quant_workspace_bytes(int, int, int, int, int) { return 0; }
extern "C" int mstf_value_spmv_quant(void*, const uint64_t*, const uint32_t*, const uint32_t*, const uint32_t*, const uint32_t*, const mstf_half*, const mstf_half*, const mstf_half*, mstf_half*, int, int, int, int, int, int, int, int, void*, size_t) { return MSTF_EUNSUPPORTED; }
