// Host-side pieces of libmiq: error reporting and the double-precision encoding arithmetic that the reference does
// on the host (ModelOptimizations/DlQuantization/src/TensorQuantizationSim.cpp:62-92,
// ModelOptimizations/DlQuantization/src/quantization_utils.cpp:58-156).
#include "miq_common.h"
#include "miq_encoding_math.h"

#include <algorithm>
#include <cmath>
#include <limits>

namespace miq
{
static thread_local char g_err[512] = "";

void set_error(const char* fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}
}   // namespace miq

extern "C" {

const char* miq_last_error(void)
{
    return miq::g_err;
}

int miq_version(void)
{
    return 1;
}

int miq_fill_encoding_info(int bw, double enc_min, double enc_max, miq_encoding* out)
{
    MIQ_CHECK_ARG(out != nullptr, "null output encoding");
    MIQ_CHECK_ARG(bw >= 1 && bw <= 32, "bitwidth must be in [1, 32] (got %d)", bw);
    // gateMinMax: keep zero inside the range and the range wider than 1e-5
    double lo = std::min(enc_min, 0.0);
    double hi = std::max(enc_max, 0.0);
    hi        = std::max(hi, lo + 1e-5);
    // strict-symmetric grids (min == -max) use one step less
    double steps = std::pow(2.0, bw) - 1;
    if (lo == -hi)
        steps -= 1;
    const double delta  = (hi - lo) / steps;
    const double offset = std::round(lo / delta);
    out->bw             = bw;
    out->delta          = delta;
    out->offset         = offset;
    out->min            = offset * delta;
    out->max            = delta * steps + out->min;
    return MIQ_OK;
}

int miq_get_computed_encodings(int bw, double mn, double mx, int use_symmetric, int use_strict_symmetric,
                               int use_unsigned_symmetric, miq_encoding* out)
{
    MIQ_CHECK_ARG(out != nullptr, "null output encoding");
    MIQ_CHECK_ARG(bw >= 1 && bw <= 32, "bitwidth must be in [1, 32] (got %d)", bw);
    const miq::EncodingD e =
        miq::computed_encodings(bw, mn, mx, use_symmetric != 0, use_strict_symmetric != 0, use_unsigned_symmetric != 0);
    out->bw     = bw;
    out->min    = e.min;
    out->max    = e.max;
    out->delta  = e.delta;
    out->offset = e.offset;
    return MIQ_OK;
}

}   // extern "C"
