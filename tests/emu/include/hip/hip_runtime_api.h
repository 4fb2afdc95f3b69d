// The host-only half of the HIP runtime header, for the emulated build: the same stand-in.
#pragma once
#include <hip/hip_runtime.h>
