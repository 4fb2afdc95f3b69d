// Version of the Thrust API surface mirrored by the cdna4 device system (thrust/version.h:50).
#pragma once
#include <thrust/system/cdna4/detail/core.h>
#define THRUST_MAJOR_VERSION (THRUST_VERSION / 100000)
#define THRUST_MINOR_VERSION (THRUST_VERSION / 100 % 1000)
#define THRUST_SUBMINOR_VERSION (THRUST_VERSION % 100)
#define THRUST_PATCH_NUMBER 0
// Set by these headers only: lets user code (and the tests) assert that <thrust/...> did not
// resolve to another Thrust installed on the include path.
#define THRUST_CDNA4_VERSION 100
