#include "ksmm_common.h"
namespace ksmm {
int wave_run(const Problem &, int, bool, ksmm_tile *) { return KSMM_ERR_BAD_ALGO; }
}
