// Same include name as the reference tree; the declarations live in nixl_sb_api.h.
#include "../nixl_sb_api.h"
