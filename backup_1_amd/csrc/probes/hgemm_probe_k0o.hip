// measurement variants of the large fp16 tile kernel: see hgemm_probe_impl.hpp
#include "hgemm_probe_impl.hpp"
namespace decx_hip_probe {
DECX_PROBE_DEFINE(probe_kind0_orders, Shape2x64, false, 16, 32, 23, 39)
}
