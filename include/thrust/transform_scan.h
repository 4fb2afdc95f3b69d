// thrust::transform_inclusive_scan / transform_exclusive_scan (thrust/transform_scan.h): a scan
// of unary_op(x) read through a transform iterator, so nothing is materialised
// (thrust/system/cuda/detail/transform_scan.h does the same).
#pragma once
#include <thrust/iterator/transform_iterator.h>
#include <thrust/scan.h>

namespace thrust {
namespace detail {
template <class Policy, class In, class Out, class UnaryOp, class BinaryOp>
Out composed_transform_inclusive_scan(const Policy& exec, In first, In last, Out result, UnaryOp unary_op, BinaryOp binary_op) {
  return inclusive_scan(exec, make_transform_iterator(first, unary_op), make_transform_iterator(last, unary_op), result, binary_op);
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class Out, class UnaryOp, class BinaryOp>
Out transform_inclusive_scan(execution_policy<D_>& exec, In first, In last, Out result, UnaryOp unary_op, BinaryOp binary_op) { return thrust::detail::composed_transform_inclusive_scan(exec, first, last, result, unary_op, binary_op); }
}}  // namespace system::cdna4
template <class D_, class In, class Out, class UnaryOp, class BinaryOp>
Out transform_inclusive_scan(const detail::execution_policy_base<D_>& exec, In first, In last, Out result, UnaryOp unary_op, BinaryOp binary_op) { return transform_inclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result, unary_op, binary_op); }
template <class In, class Out, class UnaryOp, class BinaryOp>
Out transform_inclusive_scan(const system::cpp::detail::par_t& exec, In first, In last, Out result, UnaryOp unary_op, BinaryOp binary_op) { return detail::composed_transform_inclusive_scan(exec, first, last, result, unary_op, binary_op); }
namespace detail {
template <class Policy, class In, class Out, class UnaryOp, class T, class BinaryOp>
Out composed_transform_exclusive_scan(const Policy& exec, In first, In last, Out result, UnaryOp unary_op, T init, BinaryOp binary_op) {
  return exclusive_scan(exec, make_transform_iterator(first, unary_op), make_transform_iterator(last, unary_op), result, init, binary_op);
}
}  // namespace detail
namespace system { namespace cdna4 {
template <class D_, class In, class Out, class UnaryOp, class T, class BinaryOp>
Out transform_exclusive_scan(execution_policy<D_>& exec, In first, In last, Out result, UnaryOp unary_op, T init, BinaryOp binary_op) { return thrust::detail::composed_transform_exclusive_scan(exec, first, last, result, unary_op, init, binary_op); }
}}  // namespace system::cdna4
template <class D_, class In, class Out, class UnaryOp, class T, class BinaryOp>
Out transform_exclusive_scan(const detail::execution_policy_base<D_>& exec, In first, In last, Out result, UnaryOp unary_op, T init, BinaryOp binary_op) { return transform_exclusive_scan(detail::derived_cast(detail::strip_const(exec)), first, last, result, unary_op, init, binary_op); }
template <class In, class Out, class UnaryOp, class T, class BinaryOp>
Out transform_exclusive_scan(const system::cpp::detail::par_t& exec, In first, In last, Out result, UnaryOp unary_op, T init, BinaryOp binary_op) { return detail::composed_transform_exclusive_scan(exec, first, last, result, unary_op, init, binary_op); }
template <class In, class Out, class U, class B, detail::enable_if_device<In, Out, U, B> = 0>
Out transform_inclusive_scan(In f, In l, Out o, U u, B b) { return transform_inclusive_scan(typename detail::implicit_policy<In, Out, U, B>::type(), f, l, o, u, b); }
template <class In, class Out, class U, class B, detail::enable_if_host<In, Out, U, B> = 0>
Out transform_inclusive_scan(In f, In l, Out o, U u, B b) { return transform_inclusive_scan(host, f, l, o, u, b); }
template <class In, class Out, class U, class T, class B, detail::enable_if_device<In, Out, U, T, B> = 0>
Out transform_exclusive_scan(In f, In l, Out o, U u, T init, B b) { return transform_exclusive_scan(typename detail::implicit_policy<In, Out, U, T, B>::type(), f, l, o, u, init, b); }
template <class In, class Out, class U, class T, class B, detail::enable_if_host<In, Out, U, T, B> = 0>
Out transform_exclusive_scan(In f, In l, Out o, U u, T init, B b) { return transform_exclusive_scan(host, f, l, o, u, init, b); }
}  // namespace thrust
