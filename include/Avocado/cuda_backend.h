/* Forwarding header: lets sources written against the reference (`#include <Avocado/cuda_backend.h>`) build unchanged
 * against the hot-path subset this library implements. */
#include "../avocado_hip_backend.h"
