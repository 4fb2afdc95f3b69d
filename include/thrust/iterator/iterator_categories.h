// Iterator traversal tags and the device / host iterator category tags
// (thrust/iterator/iterator_categories.h, thrust/iterator/detail/iterator_traversal_tags.h).  A
// device category derives from the standard category of the same strength, so the standard's
// algorithms accept it, and from a marker by which the algorithms of this library know that the
// iterator walks device memory.
#pragma once
#include <iterator>
#include <thrust/device_ptr.h>
namespace thrust {
struct no_traversal_tag {};
struct incrementable_traversal_tag : no_traversal_tag {};
struct single_pass_traversal_tag : incrementable_traversal_tag {};
struct forward_traversal_tag : single_pass_traversal_tag {};
struct bidirectional_traversal_tag : forward_traversal_tag {};
struct random_access_traversal_tag : bidirectional_traversal_tag {};

struct input_device_iterator_tag : std::input_iterator_tag, system::cdna4::detail::device_category_marker {};
struct output_device_iterator_tag : std::output_iterator_tag, system::cdna4::detail::device_category_marker {};
struct forward_device_iterator_tag : std::forward_iterator_tag, system::cdna4::detail::device_category_marker {};
struct bidirectional_device_iterator_tag : std::bidirectional_iterator_tag, system::cdna4::detail::device_category_marker {};
struct random_access_device_iterator_tag : std::random_access_iterator_tag, system::cdna4::detail::device_category_marker {};
typedef std::input_iterator_tag input_host_iterator_tag;
typedef std::output_iterator_tag output_host_iterator_tag;
typedef std::forward_iterator_tag forward_host_iterator_tag;
typedef std::bidirectional_iterator_tag bidirectional_host_iterator_tag;
typedef std::random_access_iterator_tag random_access_host_iterator_tag;

namespace detail {
// the standard category of a traversal tag (or of a standard category given in its place)
template <class Traversal, bool Device> struct category_of_traversal {
  typedef typename std::conditional<
      std::is_convertible<Traversal, random_access_traversal_tag>::value || std::is_convertible<Traversal, std::random_access_iterator_tag>::value,
      typename std::conditional<Device, random_access_device_iterator_tag, std::random_access_iterator_tag>::type,
      typename std::conditional<
          std::is_convertible<Traversal, bidirectional_traversal_tag>::value || std::is_convertible<Traversal, std::bidirectional_iterator_tag>::value,
          typename std::conditional<Device, bidirectional_device_iterator_tag, std::bidirectional_iterator_tag>::type,
          typename std::conditional<
              std::is_convertible<Traversal, forward_traversal_tag>::value || std::is_convertible<Traversal, std::forward_iterator_tag>::value,
              typename std::conditional<Device, forward_device_iterator_tag, std::forward_iterator_tag>::type,
              typename std::conditional<Device, input_device_iterator_tag, std::input_iterator_tag>::type>::type>::type>::type type;
};
}  // namespace detail
}  // namespace thrust
