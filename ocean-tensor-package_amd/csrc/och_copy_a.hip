/* Converting copies whose source type is one of: obool, uint8_t, uint16_t. */
#include "och_copy_tmpl.h"
namespace och { OCH_COPY_LOOKUP(a, obool, uint8_t, uint16_t) }
