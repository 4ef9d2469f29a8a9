// The vector types and short integer names of the library at global scope, as user code of the Fused Kernel Library
// expects them (its own core/data/vector_types.h defines them there).  Included by the headers under
// include/fused_kernel/ only; code that includes fk/ headers directly keeps them inside namespace fk.
#ifndef FK_CORE_GLOBAL_TYPES_H
#define FK_CORE_GLOBAL_TYPES_H

#include "fk/core/constexpr_cmath.h"
#include "fk/core/vector_types.h"

namespace cxp = fk::cxp;

using fk::uchar;
using fk::ushort;
using fk::uint;
using fk::ulong;
using fk::longlong;
using fk::ulonglong;
using fk::bool1; using fk::bool2; using fk::bool3; using fk::bool4;
using fk::char1; using fk::char2; using fk::char3; using fk::char4;
using fk::uchar1; using fk::uchar2; using fk::uchar3; using fk::uchar4;
using fk::short1; using fk::short2; using fk::short3; using fk::short4;
using fk::ushort1; using fk::ushort2; using fk::ushort3; using fk::ushort4;
using fk::int1; using fk::int2; using fk::int3; using fk::int4;
using fk::uint1; using fk::uint2; using fk::uint3; using fk::uint4;
using fk::long1; using fk::long2; using fk::long3; using fk::long4;
using fk::ulong1; using fk::ulong2; using fk::ulong3; using fk::ulong4;
using fk::longlong1; using fk::longlong2; using fk::longlong3; using fk::longlong4;
using fk::ulonglong1; using fk::ulonglong2; using fk::ulonglong3; using fk::ulonglong4;
using fk::float1; using fk::float2; using fk::float3; using fk::float4;
using fk::double1; using fk::double2; using fk::double3; using fk::double4;

#endif
