/* Forwarding header: lets sources written against the reference (`#include <Avocado/backend_defs.h>`) build unchanged. */
#include "../avocado_backend_defs.h"
