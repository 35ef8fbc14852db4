#include "context.hpp"
struct pcmm_ctx;
namespace ckks {
struct PpmmArgs;
int launch_ppmm_mfma(pcmm_ctx*, const PpmmArgs&, int, int) { set_error("PPMM MFMA path not built"); return CKKS_E_INVALID; }
}
