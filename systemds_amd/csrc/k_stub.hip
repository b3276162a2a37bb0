// Placeholders for drivers whose kernels are not written yet: they fail loudly.
#include "../../include/cla_hip.h"
#include "cla_internal.hpp"
namespace cla {
#define NOT_YET(name) do { set_error(name ": not implemented"); return -CLA_ERR_UNSUPPORTED; } while(0)
int launch_decompress(cla_block*, double*, unsigned long long*) { NOT_YET("decompress"); }
int launch_tsmm(cla_block*, double*, unsigned long long*) { NOT_YET("tsmm"); }
int launch_cooc(cla_block*, int, int, unsigned long long*) { NOT_YET("cooc"); }
}
