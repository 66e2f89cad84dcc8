/* Converting copies whose source type is one of: uint32_t, uint64_t, int8_t. */
#include "och_copy_tmpl.h"
namespace och { OCH_COPY_LOOKUP(b, uint32_t, uint64_t, int8_t) }
