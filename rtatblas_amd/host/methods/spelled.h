// Problem keys and variant descriptors are identified by their spelling: the text is what
// they are ordered by in the planner's maps, what they print as, and (for variants) what a
// stream reader parses.  A type states its spelling once and inherits the rest from here.
#pragma once
#include <istream>
#include <ostream>
#include <string>
#include <tuple>
#include <type_traits>
#include <utility>
#include <vector>

namespace rtat {

// D provides `std::string text() const`.  Ordering is lexicographic on the text — the same
// order the reference's keys and variants have (e.g. gemm.cpp:18-20), so maps and the JSON
// reports built from them iterate alike.
template <class D>
struct Spelled {
  operator std::string() const { return static_cast<const D&>(*this).text(); }
  friend bool operator<(const D& a, const D& b) { return a.text() < b.text(); }
  friend std::ostream& operator<<(std::ostream& os, const D& d) { return os << d.text(); }
};

// A problem key: its fields never change after construction, so the spelling is built once
// and every later comparison is a plain string compare without allocation.  D passes the
// finished text to the constructor.
template <class D>
class Spelled_Once {
  std::string label;

 protected:
  explicit Spelled_Once(std::string text) : label(std::move(text)) {}

 public:
  const std::string& text() const { return label; }
  operator std::string() const { return label; }
  friend bool operator<(const D& a, const D& b) { return a.text() < b.text(); }
  friend std::ostream& operator<<(std::ostream& os, const D& d) { return os << d.text(); }
};

namespace detail {
// Switches with multi-letter names declare `static constexpr bool named = true`.
template <class Switch, class = void>
struct is_named_switch : std::false_type {};
template <class Switch>
struct is_named_switch<Switch, std::enable_if_t<Switch::named>> : std::true_type {};
}  // namespace detail

// A variant made of independent switches (BLAS_Op, Pad_Op, Bool_Op, Tile_Op ...).  D provides
// `auto switches()` / `auto switches() const`: a std::tie of its switch members in spelling
// order, the one-letter switches first.  From that follow
//   * text():       the one-letter switches back to back, then each named switch behind a
//                   slash ("TNN", "FT", "NNTNPN", "NNN/128x64", "FF/auto/split/1024");
//   * enumerate():  every setting, first switch slowest ("NNN NNT NTN ...");
//   * spell_into(): the inverse of text(), false when the text has the wrong shape.
template <class D>
struct Switch_Variant : Spelled<D> {
  static D default_opts() { return D(); }

  std::string text() const {
    std::string out;
    std::apply(
        [&](const auto&... sw) {
          ((out += (detail::is_named_switch<std::decay_t<decltype(sw)>>::value ? "/" : "") +
                   std::string(sw)),
           ...);
        },
        static_cast<const D&>(*this).switches());
    return out;
  }

  static std::vector<D> enumerate() {
    std::vector<D> settings{D()};
    vary<0>(settings);
    return settings;
  }

  // Sets every switch from its part of the text: one letter each for the leading switches,
  // one slash-separated name each for the named ones.  A text of the wrong shape (length of
  // the letter part, number of names) leaves `d` alone and returns false; a letter or name
  // that spells nothing throws, as the switch types themselves do.
  static bool spell_into(D& d, const std::string& text) {
    std::vector<std::string> parts;  // [letters, name, name, ...]
    size_t from = 0;
    for (size_t at; (at = text.find('/', from)) != std::string::npos; from = at + 1)
      parts.push_back(text.substr(from, at - from));
    parts.push_back(text.substr(from));
    size_t letters = 0, names = 0;
    D fresh;
    std::apply(
        [&](auto&... sw) {
          ((detail::is_named_switch<std::decay_t<decltype(sw)>>::value ? ++names : ++letters), ...);
        },
        fresh.switches());
    if (parts.size() != names + 1 || parts[0].size() != letters) return false;
    size_t at = 0, name = 1;
    std::apply(
        [&](auto&... sw) {
          (([&] {
             using Switch = std::decay_t<decltype(sw)>;
             if constexpr (detail::is_named_switch<Switch>::value) sw = Switch(parts[name++]);
             else sw = Switch(parts[0][at++]);
           }()),
           ...);
        },
        fresh.switches());
    d = fresh;
    return true;
  }

  friend std::istream& operator>>(std::istream& is, D& d) {
    std::string word;
    is >> word;
    if (!D::spell_into(d, word)) is.setstate(std::ios::failbit);
    return is;
  }

 private:
  template <size_t I>
  static void vary(std::vector<D>& settings) {
    if constexpr (I < std::tuple_size_v<decltype(std::declval<D&>().switches())>) {
      using Switch = std::remove_reference_t<decltype(std::get<I>(std::declval<D&>().switches()))>;
      std::vector<D> widened;
      for (const D& d : settings)
        for (const Switch& value : Switch::enumerate()) {
          D e = d;
          std::get<I>(e.switches()) = value;
          widened.push_back(e);
        }
      settings.swap(widened);
      vary<I + 1>(settings);
    }
  }
};

}  // namespace rtat
