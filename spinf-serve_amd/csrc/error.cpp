#include "spinf_tree.h"
#include "common.h"

static thread_local char g_err[512] = "";

int spinf_fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

extern "C" const char* spinf_last_error(void) { return g_err; }
extern "C" int spinf_version(void) { return 1; }

// sizeof of the argument blocks, in the order of their declaration: what a binding in another language checks its own mirror of
// the structures against before the first call
extern "C" int spinf_struct_sizes(int64_t* sizes, int32_t n) {
    const int64_t all[7] = {(int64_t)sizeof(spinf_attn_args), (int64_t)sizeof(spinf_gdn_args), (int64_t)sizeof(spinf_gdn_pre_args),
                            (int64_t)sizeof(spinf_gdn_gate_args), (int64_t)sizeof(spinf_lm_args), (int64_t)sizeof(spinf_lm_head_args),
                            (int64_t)sizeof(spinf_xdec_args)};
    if (!sizes || n != 7) return spinf_fail(SPINF_E_ARG, "struct_sizes: 7 sizes (attn, gdn, gdn_pre, gdn_gate, lm, lm_head, xdec)");
    for (int i = 0; i < 7; i++) sizes[i] = all[i];
    return SPINF_OK;
}
