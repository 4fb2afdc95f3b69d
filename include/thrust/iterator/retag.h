// thrust::retag / reinterpret_tag (thrust/iterator/retag.h): the same iterator, declared to walk
// the memory of another system — retag<thrust::device_system_tag>(raw_pointer) makes a range the
// algorithms treat as device memory.
#pragma once
#include <thrust/iterator/iterator_adaptor.h>
namespace thrust {
namespace detail {
template <class Iterator, class Tag>
class tagged_iterator : public iterator_adaptor<tagged_iterator<Iterator, Tag>, Iterator, use_default, Tag> {
  typedef iterator_adaptor<tagged_iterator<Iterator, Tag>, Iterator, use_default, Tag> super_t;
 public:
  tagged_iterator() = default;
  THRUST_CDNA4_HD explicit tagged_iterator(Iterator it) : super_t(it) {}
};
}  // namespace detail
template <class Tag, class Iterator>
THRUST_CDNA4_HD detail::tagged_iterator<Iterator, Tag> reinterpret_tag(Iterator iter) { return detail::tagged_iterator<Iterator, Tag>(iter); }
// a device pointer stays one under a tag of the device system (its reference type reads and writes
// device memory from the host); under any other tag it is the raw address
template <class Tag, class T, typename std::enable_if<std::is_convertible<Tag, device_system_tag>::value, int>::type = 0>
THRUST_CDNA4_HD detail::tagged_iterator<device_ptr<T>, Tag> reinterpret_tag(device_ptr<T> iter) { return detail::tagged_iterator<device_ptr<T>, Tag>(iter); }
template <class Tag, class T, typename std::enable_if<!std::is_convertible<Tag, device_system_tag>::value, int>::type = 0>
THRUST_CDNA4_HD detail::tagged_iterator<T*, Tag> reinterpret_tag(device_ptr<T> iter) { return detail::tagged_iterator<T*, Tag>(iter.get()); }
template <class Tag, class Iterator>
THRUST_CDNA4_HD auto retag(Iterator iter) -> decltype(reinterpret_tag<Tag>(iter)) { return reinterpret_tag<Tag>(iter); }
}  // namespace thrust
