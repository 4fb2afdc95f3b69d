// <thrust/memory.h>: pointer casts and raw memory helpers for the device system
// (raw_pointer_cast, raw_reference_cast, device_malloc / device_free through the pool).
#pragma once
#include <thrust/detail/raw_reference_cast.h>
#include <thrust/device_free.h>
#include <thrust/device_malloc.h>
#include <thrust/device_ptr.h>
