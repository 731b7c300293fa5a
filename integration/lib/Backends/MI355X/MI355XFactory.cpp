/**
 * Registers the MI355X backend with Glow's backend factory
 * (include/glow/Backend/Backend.h:341-356; lib/Backends/CPU/CPUFactory.cpp).
 * NOT COMPILED in the repository this file ships in.
 */
#include "MI355XBackend.h"

namespace glow {

REGISTER_GLOW_BACKEND_FACTORY(MI355XFactory, MI355XBackend);

} // namespace glow
