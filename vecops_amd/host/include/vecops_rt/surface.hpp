// Selects the runtime surface the HIP plug-in is compiled against: the restated
// one of this repository (default) or the vecops tree's own headers.  The plug-in
// sources use only names both provide.
#ifndef VECOPS_RT_SURFACE_HPP
#define VECOPS_RT_SURFACE_HPP

#ifdef VECOPS_HIP_USE_UPSTREAM_RUNTIME
#include "vecops/runtime/Executable.h"
#include "vecops/runtime/KernelDefinition.h"
#include "vecops/runtime/Operator.h"
#include "vecops/runtime/OperatorBridgeAbi.h"
#include "vecops/runtime/Schema.h"
#include "vecops/runtime/Status.h"
#else
#include "vecops_rt/runtime.hpp"
#endif

#endif
