// TEST INFRASTRUCTURE.  Stands where the reference's utils/DataLoader.h stands
// when the reference tree is not available; the loader itself is the
// repository's own (include/swc_host_utils.h).
#pragma once
#include "swc_host_utils.h"
