// measurement variants of the large fp16 tile kernel: see hgemm_probe_impl.hpp
#include "hgemm_probe_impl.hpp"
namespace decx_hip_probe {
DECX_PROBE_DEFINE(probe_kind5, ShapeFat, false, 0, 4, 5, 7, 12)
}
