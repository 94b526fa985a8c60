// The traversal tags iterators built on thrust::iterator_facade name, and the category tags of the
// two systems (thrust/iterator/iterator_categories.h:50-190, detail/iterator_traversal_tags.h).
// The host categories are the standard's; a device category is the standard's under another name,
// since the system of an iterator is told by thrust::iterator_system here, not by its category.
#pragma once
#include <iterator>

namespace thrust {
struct incrementable_traversal_tag {};
struct single_pass_traversal_tag : incrementable_traversal_tag {};
struct forward_traversal_tag : single_pass_traversal_tag {};
struct bidirectional_traversal_tag : forward_traversal_tag {};
struct random_access_traversal_tag : bidirectional_traversal_tag {};

typedef std::input_iterator_tag input_host_iterator_tag;
typedef std::output_iterator_tag output_host_iterator_tag;
typedef std::forward_iterator_tag forward_host_iterator_tag;
typedef std::bidirectional_iterator_tag bidirectional_host_iterator_tag;
typedef std::random_access_iterator_tag random_access_host_iterator_tag;
struct input_device_iterator_tag : std::input_iterator_tag {};
struct output_device_iterator_tag : std::output_iterator_tag {};
struct forward_device_iterator_tag : std::forward_iterator_tag {};
struct bidirectional_device_iterator_tag : std::bidirectional_iterator_tag {};
struct random_access_device_iterator_tag : std::random_access_iterator_tag {};

namespace detail {
// the standard category that allows what a traversal tag allows
template <typename Traversal> struct category_of_traversal { typedef Traversal type; };  // a standard tag already
template <> struct category_of_traversal<incrementable_traversal_tag> { typedef std::output_iterator_tag type; };
template <> struct category_of_traversal<single_pass_traversal_tag> { typedef std::input_iterator_tag type; };
template <> struct category_of_traversal<forward_traversal_tag> { typedef std::forward_iterator_tag type; };
template <> struct category_of_traversal<bidirectional_traversal_tag> { typedef std::bidirectional_iterator_tag type; };
template <> struct category_of_traversal<random_access_traversal_tag> { typedef std::random_access_iterator_tag type; };
}  // namespace detail
}  // namespace thrust
