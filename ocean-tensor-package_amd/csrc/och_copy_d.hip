/* Converting copies whose source type is one of: half_t, float, double. */
#include "och_copy_tmpl.h"
namespace och { OCH_COPY_LOOKUP(d, half_t, float, double) }
