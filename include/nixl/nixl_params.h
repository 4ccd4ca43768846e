// Same include name as the reference tree; the declarations live in nixl_nb_api.h.
#include "nixl_nb_api.h"
