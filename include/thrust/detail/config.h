// <thrust/detail/config.h>: configuration macros user code tests (device system, namespace).
#pragma once
#include <thrust/version.h>
#ifndef THRUST_NAMESPACE_BEGIN
#define THRUST_NAMESPACE_BEGIN namespace thrust {
#define THRUST_NAMESPACE_END }
#endif
#ifndef THRUST_PREVENT_MACRO_SUBSTITUTION
#define THRUST_PREVENT_MACRO_SUBSTITUTION
#endif
