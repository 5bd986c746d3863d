// TEST INFRASTRUCTURE ONLY — execution switch of the CPU restatement.
#include <omp.h>

#include "common.hpp"

namespace orc {
static int g_threads = 1;
int num_threads() { return g_threads; }
}  // namespace orc

// 1 (default) = sequential and deterministic; n > 1 = the reference's parallel decomposition
// on n OpenMP threads; 0 = all hardware threads.  Returns the value now in force.
extern "C" int oracle_set_num_threads(int n) {
    if (n <= 0) n = omp_get_num_procs();
    orc::g_threads = n;
    return n;
}
extern "C" int oracle_get_num_threads() { return orc::g_threads; }
