// thrust::iterator_adaptor (thrust/iterator/iterator_adaptor.h): an iterator built around
// another one.  The derived class overrides the core functions it wants to change (most often
// dereference()); everything else forwards to the base iterator.  Template arguments left at
// use_default come from the base iterator: its value type, its reference, its difference type, its
// traversal, and the system of the memory it walks.
#pragma once
#include <iterator>
#include <type_traits>
#include <thrust/iterator/iterator_facade.h>
#include <thrust/iterator/iterator_traits.h>
namespace thrust {
namespace detail {
template <class T, class Default> struct or_default { typedef T type; };
template <class Default> struct or_default<use_default, Default> { typedef Default type; };
template <class Base> struct system_of_base {
  typedef typename std::conditional<system::cdna4::detail::is_device_iterator<Base>::value, device_system_tag, host_system_tag>::type type;
};
}  // namespace detail

template <class Derived, class Base, class Value = use_default, class System = use_default, class Traversal = use_default,
          class Reference = use_default, class Difference = use_default>
class iterator_adaptor
    : public iterator_facade<Derived, typename detail::or_default<Value, typename std::iterator_traits<Base>::value_type>::type,
                             typename detail::or_default<System, typename detail::system_of_base<Base>::type>::type,
                             typename detail::or_default<Traversal, typename std::iterator_traits<Base>::iterator_category>::type,
                             typename detail::or_default<
                                 Reference, typename std::conditional<std::is_same<Value, use_default>::value, typename std::iterator_traits<Base>::reference,
                                                                      typename std::add_lvalue_reference<Value>::type>::type>::type,
                             typename detail::or_default<Difference, typename std::iterator_traits<Base>::difference_type>::type> {
  friend class iterator_core_access;
 public:
  typedef Base base_type;
  typedef iterator_adaptor super_t;  // what derived classes name their base, as in the reference
  typedef typename iterator_adaptor::iterator_facade facade_type;
  typedef typename facade_type::reference reference;
  typedef typename facade_type::difference_type difference_type;
  iterator_adaptor() = default;
  THRUST_CDNA4_HD explicit iterator_adaptor(const Base& iter) : m_iterator(iter) {}
  THRUST_CDNA4_HD const Base& base() const { return m_iterator; }
 protected:
  THRUST_CDNA4_HD const Base& base_reference() const { return m_iterator; }
  THRUST_CDNA4_HD Base& base_reference() { return m_iterator; }
 private:
  THRUST_CDNA4_HD reference dereference() const { return *m_iterator; }
  template <class O> THRUST_CDNA4_HD bool equal(const O& other) const { return m_iterator == other.base(); }
  THRUST_CDNA4_HD void advance(difference_type n) { m_iterator += n; }
  THRUST_CDNA4_HD void increment() { ++m_iterator; }
  THRUST_CDNA4_HD void decrement() { --m_iterator; }
  template <class O> THRUST_CDNA4_HD difference_type distance_to(const O& other) const { return other.base() - m_iterator; }
  Base m_iterator;
};
}  // namespace thrust
