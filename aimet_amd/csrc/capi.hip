// Entry points that do not belong to one kernel family.
#include "ahq_host.h"

extern "C" const char* ahq_last_error(void) { return ahq::error_buffer(); }
extern "C" int ahq_version(void) { return 1; }
