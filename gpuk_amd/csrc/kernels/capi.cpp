// Entry points of the C ABI that launch nothing: status names, version, tuning knobs.
#include <string.h>

#include "../../../include/gpuk_amd.h"
#include "host_utils.h"

extern "C" const char *gpuk_status_string(int status) {
    switch (status) {
        case GPUK_OK: return "ok";
        case GPUK_ERR_INVALID_ARG: return "invalid argument";
        case GPUK_ERR_UNSUPPORTED: return "unsupported shape, dtype or mode";
        case GPUK_ERR_MISALIGNED: return "pointer not aligned for vector access";
        case GPUK_ERR_LAUNCH: return "kernel launch failed";
        case GPUK_ERR_INTERNAL: return "internal error";
        default: return "unknown status";
    }
}

extern "C" int gpuk_abi_version(void) { return GPUK_AMD_ABI_VERSION; }

extern "C" int gpuk_set_tuning(const char *key, int value) {
    if (!key) return GPUK_ERR_INVALID_ARG;
    if (strcmp(key, "norm_quant_nchunk") == 0) {
        if (value != 0 && value != 1 && value != 2 && value != 4 && value != 8) return GPUK_ERR_INVALID_ARG;
        gpuk::set_norm_quant_tuning(0, value);
        return GPUK_OK;
    }
    if (strcmp(key, "norm_quant_threads") == 0) {
        if (value < 0 || value > 1024 || value % 64) return GPUK_ERR_INVALID_ARG;
        gpuk::set_norm_quant_tuning(1, value);
        return GPUK_OK;
    }
    if (strcmp(key, "norm_quant_row_group_shift") == 0) {  // -1 = heuristic, 0..10
        if (value < -1 || value > 10) return GPUK_ERR_INVALID_ARG;
        gpuk::set_norm_quant_tuning(5, value);
        return GPUK_OK;
    }
    if (strcmp(key, "norm_quant_gate") == 0) {  // ticks of 10 ns; -1 = built-in rule, 0 = no gate
        if (value < -1 || value > 5000) return GPUK_ERR_INVALID_ARG;
        gpuk::set_norm_quant_tuning(6, value);
        return GPUK_OK;
    }
    if (strcmp(key, "norm_quant_launches") == 0) {  // 0 = built-in rule, 1 = always one, 2 = two wherever each half fits a round
        if (value < 0 || value > 2) return GPUK_ERR_INVALID_ARG;
        gpuk::set_norm_quant_tuning(7, value);
        return GPUK_OK;
    }
    if (strcmp(key, "rope_unit_gate") == 0) {
        if (value < -1 || value > 5000) return GPUK_ERR_INVALID_ARG;
        gpuk::set_rope_tuning(6, value);
        return GPUK_OK;
    }
    if (strcmp(key, "rope_token_waves") == 0) {
        if (value < 0 || value > 3) return GPUK_ERR_INVALID_ARG;
        gpuk::set_rope_tuning(1, value);
        return GPUK_OK;
    }
    if (strcmp(key, "rope_token_gate") == 0) {  // ticks of 10 ns; -1 = from the bytes of the call
        if (value < -1 || value > 5000) return GPUK_ERR_INVALID_ARG;
        gpuk::set_rope_tuning(2, value);
        return GPUK_OK;
    }
    if (strcmp(key, "rope_stream_rows") == 0) {
        if (value < 0 || value > 2) return GPUK_ERR_INVALID_ARG;
        gpuk::set_rope_tuning(3, value);
        return GPUK_OK;
    }
    if (strcmp(key, "rope_merge_rows") == 0) {
        if (value < 0 || value > 1) return GPUK_ERR_INVALID_ARG;
        gpuk::set_rope_tuning(4, value);
        return GPUK_OK;
    }
    if (strcmp(key, "rope_block_threads") == 0) {
        if (value != 0 && value != 64 && value != 128 && value != 256 && value != 512) return GPUK_ERR_INVALID_ARG;
        gpuk::set_rope_tuning(0, value);
        return GPUK_OK;
    }
    return GPUK_ERR_INVALID_ARG;
}
