// Entry points that carry no kernel: version and error text.
#include "k3q_common.h"

extern "C" int k3q_version(void) { return 100; }

extern "C" const char* k3q_error_string(int code) {
    switch (code) {
        case K3Q_OK: return "ok";
        case K3Q_ERR_NULL: return "a required pointer is null";
        case K3Q_ERR_SHAPE: return "negative, zero or inconsistent extent";
        case K3Q_ERR_ALIGN: return "pointer or stride breaks the required alignment";
        case K3Q_ERR_DTYPE: return "unknown dtype code";
        case K3Q_ERR_WORKSPACE: return "workspace missing or too small";
        case K3Q_ERR_LAUNCH: return "the HIP runtime refused the kernel launch";
        case K3Q_ERR_RANGE: return "value range does not fit the output dtype";
        default: return "unknown k3q error code";
    }
}
