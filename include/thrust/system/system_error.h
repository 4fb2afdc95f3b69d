// thrust::system::system_error (thrust/system/system_error.h): the exception every failed device
// call turns into, carrying the hip error code in the cdna4 category.
#pragma once
#include <thrust/system/error_code.h>
#include <thrust/system_error.h>
namespace thrust { namespace system {
using ::thrust::system_error;
}}  // namespace thrust::system
