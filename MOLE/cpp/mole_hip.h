/* The C ABI lives in include/mole_hip.h at the repository root; this file puts it where the reference keeps
 * its native sources (MOLE/cpp). */
#include "../../include/mole_hip.h"
