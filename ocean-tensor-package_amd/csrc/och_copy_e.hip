/* Converting copies whose source type is one of: chalf_t, cfloat_t, cdouble_t. */
#include "och_copy_tmpl.h"
namespace och { OCH_COPY_LOOKUP(e, chalf_t, cfloat_t, cdouble_t) }
