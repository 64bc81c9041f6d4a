// Boolean predicates and their combinations, used to say which variants may be tried for
// which problems (reference src/methods/predicates.h).
#pragma once
#include <algorithm>
#include <functional>
#include <vector>

namespace rtat {

template <typename T>
using Predicate = std::function<bool(T)>;

namespace detail {
// True when `holds(p(v))` for any / all p, by the std algorithm handed in.
template <typename T, typename Quantifier>
Predicate<T> quantified(std::vector<Predicate<T>> preds, Quantifier over) {
  return [preds = std::move(preds), over](T v) {
    return over(preds.begin(), preds.end(), [&v](const Predicate<T>& p) { return p(v); });
  };
}
}  // namespace detail

// True when at least one of `preds` is (false for an empty list).
template <typename T>
Predicate<T> disjunction(std::vector<Predicate<T>> preds) {
  using It = typename std::vector<Predicate<T>>::const_iterator;
  return detail::quantified<T>(std::move(preds), [](It first, It last, auto holds) {
    return std::any_of(first, last, holds);
  });
}

// True when every one of `preds` is (true for an empty list).
template <typename T>
Predicate<T> conjunction(std::vector<Predicate<T>> preds) {
  using It = typename std::vector<Predicate<T>>::const_iterator;
  return detail::quantified<T>(std::move(preds), [](It first, It last, auto holds) {
    return std::all_of(first, last, holds);
  });
}

// True when `pred` is not.
template <typename T>
Predicate<T> negation(Predicate<T> pred) {
  return [pred = std::move(pred)](T v) { return !pred(v); };
}

}  // namespace rtat
