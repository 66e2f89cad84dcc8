/* Converting copies whose source type is one of: int16_t, int32_t, int64_t. */
#include "och_copy_tmpl.h"
namespace och { OCH_COPY_LOOKUP(c, int16_t, int32_t, int64_t) }
