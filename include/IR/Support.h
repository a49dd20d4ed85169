// Small stand-ins for the LLVM ADT / Support names that appear in the public
// headers (llvm::SmallVector, llvm::ArrayRef, llvm::StringRef, llvm::errs ...).
// The library has no LLVM dependency; these are thin wrappers over the C++
// standard library with the members the code base uses.
#pragma once

#include <cassert>
#include <cstdint>
#include <functional>
#include <initializer_list>
#include <iostream>
#include <optional>
#include <sstream>
#include <string>
#include <string_view>
#include <type_traits>
#include <vector>

namespace llvm {

template <typename T, unsigned N = 4>
class SmallVector : public std::vector<T> {
public:
  using Base = std::vector<T>;
  using Base::Base;
  SmallVector() = default;
  SmallVector(const Base& v) : Base(v) {}
  SmallVector(std::initializer_list<T> il) : Base(il) {}
  template <typename Range, typename = decltype(std::declval<const Range&>().begin()),
            typename = std::enable_if_t<!std::is_base_of<Base, std::decay_t<Range>>::value>>
  SmallVector(const Range& r) : Base(r.begin(), r.end()) {}
  template <typename It>
  void append(It b, It e) { this->insert(this->end(), b, e); }
  void append(std::initializer_list<T> il) { this->insert(this->end(), il.begin(), il.end()); }
  T pop_back_val() { T v = this->back(); this->pop_back(); return v; }
};

template <typename T>
class ArrayRef {
public:
  ArrayRef() = default;
  ArrayRef(const T* d, size_t n) : data_(d), size_(n) {}
  ArrayRef(const T& one) : data_(&one), size_(1) {}
  ArrayRef(const std::vector<T>& v) : data_(v.data()), size_(v.size()) {}
  template <unsigned N>
  ArrayRef(const SmallVector<T, N>& v) : data_(v.data()), size_(v.size()) {}
  ArrayRef(std::initializer_list<T> il) : data_(il.begin()), size_(il.size()) {}
  const T* begin() const { return data_; }
  const T* end() const { return data_ + size_; }
  const T* data() const { return data_; }
  size_t size() const { return size_; }
  bool empty() const { return size_ == 0; }
  const T& operator[](size_t i) const { assert(i < size_); return data_[i]; }
  const T& front() const { return data_[0]; }
  const T& back() const { return data_[size_ - 1]; }
  std::vector<T> vec() const { return std::vector<T>(begin(), end()); }
  ArrayRef<T> drop_front(size_t n = 1) const { return ArrayRef<T>(data_ + n, size_ - n); }
  bool operator==(const ArrayRef<T>& o) const {
    if (size_ != o.size_) return false;
    for (size_t i = 0; i < size_; ++i) if (!(data_[i] == o.data_[i])) return false;
    return true;
  }

private:
  const T* data_ = nullptr;
  size_t size_ = 0;
};

template <typename T>
ArrayRef<T> makeArrayRef(const std::vector<T>& v) { return ArrayRef<T>(v); }
template <typename T>
ArrayRef<T> makeArrayRef(std::initializer_list<T> il) { return ArrayRef<T>(il); }

// Owning string with the StringRef members the code base touches.
class StringRef {
public:
  StringRef() = default;
  StringRef(const char* s) : s_(s ? s : "") {}
  StringRef(const std::string& s) : s_(s) {}
  StringRef(std::string_view s) : s_(s) {}
  std::string str() const { return s_; }
  const char* data() const { return s_.data(); }
  size_t size() const { return s_.size(); }
  bool empty() const { return s_.empty(); }
  bool contains(const StringRef& o) const { return s_.find(o.s_) != std::string::npos; }
  bool startswith(const StringRef& o) const { return s_.rfind(o.s_, 0) == 0; }
  size_t find(const StringRef& o) const { return s_.find(o.s_); }
  operator std::string() const { return s_; }
  bool operator==(const StringRef& o) const { return s_ == o.s_; }
  bool operator!=(const StringRef& o) const { return s_ != o.s_; }
  bool operator==(const std::string& o) const { return s_ == o; }
  bool operator==(const char* o) const { return s_ == o; }
  static constexpr size_t npos = std::string::npos;

private:
  std::string s_;
};
inline std::ostream& operator<<(std::ostream& os, const StringRef& s) { return os << s.str(); }

class raw_ostream {
public:
  explicit raw_ostream(std::ostream& os) : os_(os) {}
  template <typename T>
  raw_ostream& operator<<(const T& v) { os_ << v; return *this; }
  raw_ostream& operator<<(bool v) { os_ << (v ? 1 : 0); return *this; }
  std::ostream& stream() { return os_; }
  void flush() { os_.flush(); }

private:
  std::ostream& os_;
};
inline raw_ostream& errs() { static raw_ostream s(std::cerr); return s; }
inline raw_ostream& outs() { static raw_ostream s(std::cout); return s; }

template <typename Fn>
using function_ref = std::function<Fn>;

}  // namespace llvm
