/* What host/gpu_module.c -- the GPU device module -- is compiled against.
 *
 * With OC_REFERENCE_HEADERS defined these are Ocean's own headers (-I<ocean>/include -I<ocean>/solid/include): the
 * module then uses the reference's declarations of every base-library and interface function it calls, and links
 * against Ocean's libraries as src/core/gpu does. Without it, ocean_abi.h restates the shared object layouts and
 * ocean_base.h declares the same functions, implemented by the stand-in base library host_base.c, so that the module
 * table can be driven where Ocean's libraries are not present.
 */
#ifndef OCEAN_HOST_H
#define OCEAN_HOST_H

#ifdef OC_REFERENCE_HEADERS
#include "ocean.h"
#include "ocean/external/ocean-solid/ocean_solid.h"
#else
#include "ocean_abi.h"
#include "ocean_base.h"
#endif
#include "oc_op_tables.h"
#include "../../include/ocean_gpu_module.h"

#endif
