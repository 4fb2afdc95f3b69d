// thrust::system::error_code / error_condition / error_category / errc
// (thrust/system/error_code.h): the standard's types, which the reference's are modelled on.
#pragma once
#include <system_error>
#include <thrust/system/cdna4/detail/core.h>
namespace thrust {
namespace system {
using std::error_category;
using std::error_code;
using std::error_condition;
using std::errc;
using std::generic_category;
using std::system_category;
using std::make_error_code;
using std::make_error_condition;
}  // namespace system
using system::error_condition;
using system::generic_category;
using system::system_category;
}  // namespace thrust
