// Entry points of the C ABI that are not kernels: error text, ABI revision, tuning knobs.
#include "hyc_common.hpp"

extern "C" const char* hyc_error_string(int code) {
    switch (code) {
        case HYC_OK: return "ok";
        case HYC_ERR_NULL: return "a required pointer is NULL";
        case HYC_ERR_QBIT: return "q_bit must be 2, 4 or 8";
        case HYC_ERR_SHAPE: return "invalid shape (negative or oversized dimension, or channel count not a multiple of 32)";
        case HYC_ERR_ALIGN: return "pointer or stride not aligned for 128-bit access";
        case HYC_ERR_RANK: return "unsupported LoRA rank (multiple of 4 between 4 and 64 required)";
        case HYC_ERR_LAUNCH: return "HIP kernel launch failed";
        case HYC_ERR_WORKSPACE: return "workspace too small";
        case HYC_ERR_ARG: return "invalid argument";
        default: return "unknown error code";
    }
}

extern "C" int hyc_abi_version(void) { return 11; }

extern "C" int hyc_set_tuning(const char* key, int value) {
    if (!key) return HYC_ERR_NULL;
    int rc = hyc::tune_quant(key, value);
    if (rc != 1) return rc;
    rc = hyc::tune_fuse(key, value);
    if (rc != 1) return rc;
    rc = hyc::tune_add(key, value);
    if (rc != 1) return rc;
    rc = hyc::tune_contract(key, value);
    if (rc != 1) return rc;
    rc = hyc::tune_norm_compress(key, value);
    if (rc != 1) return rc;
    rc = hyc::tune_stats(key, value);
    if (rc != 1) return rc;
    return HYC_ERR_ARG;
}
