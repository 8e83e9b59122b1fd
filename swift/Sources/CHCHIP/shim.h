/* The whole C surface the Swift backend binds: the hchip C ABI. */
#include "../../../include/hchip.h"
