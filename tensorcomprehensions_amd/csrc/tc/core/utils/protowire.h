// Minimal proto2 wire-format writer/reader (varints, bools, enums, nested messages, strings).
// The options and cache messages use nothing else, so a code generator is not needed.
#pragma once
#include <cstdint>
#include <stdexcept>
#include <string>

namespace tc {
namespace protowire {

class Writer {
 public:
  void varint(int field, uint64_t v) {
    raw((static_cast<uint64_t>(field) << 3) | 0);
    raw(v);
  }
  void boolean(int field, bool b) { varint(field, b ? 1 : 0); }
  void bytes(int field, const std::string& s) {
    raw((static_cast<uint64_t>(field) << 3) | 2);
    raw(s.size());
    out_ += s;
  }
  void fixed64(int field, uint64_t v) {
    raw((static_cast<uint64_t>(field) << 3) | 1);
    for (int i = 0; i < 8; ++i) {
      out_.push_back(static_cast<char>((v >> (8 * i)) & 0xff));
    }
  }
  const std::string& str() const { return out_; }

 private:
  void raw(uint64_t v) {
    while (v >= 0x80) {
      out_.push_back(static_cast<char>((v & 0x7f) | 0x80));
      v >>= 7;
    }
    out_.push_back(static_cast<char>(v));
  }
  std::string out_;
};

// Reads one message.  Robust against truncated or corrupt input (a cache file is untrusted
// data): every length is checked against what is left, a varint ends after ten bytes, and the
// accessors refuse a field whose wire type is not the one asked for.
class Reader {
 public:
  explicit Reader(const std::string& s) : s_(s) {}
  bool next() {
    if (pos_ >= s_.size()) {
      return false;
    }
    uint64_t key = raw();
    field_ = static_cast<int>(key >> 3);
    wire_ = static_cast<int>(key & 7);
    value_ = 0;
    bytes_.clear();
    if (wire_ == 0) {
      value_ = raw();
    } else if (wire_ == 2) {
      uint64_t n = raw();
      if (n > s_.size() - pos_) {
        throw std::runtime_error("protowire: truncated length-delimited field");
      }
      bytes_ = s_.substr(pos_, static_cast<size_t>(n));
      pos_ += static_cast<size_t>(n);
    } else if (wire_ == 1 || wire_ == 5) {
      const size_t width = wire_ == 1 ? 8 : 4;
      if (width > s_.size() - pos_) {
        throw std::runtime_error("protowire: truncated fixed-width field");
      }
      for (size_t i = 0; i < width; ++i) {
        value_ |= static_cast<uint64_t>(static_cast<unsigned char>(s_[pos_ + i])) << (8 * i);
      }
      pos_ += width;
    } else {
      throw std::runtime_error("protowire: unsupported wire type");
    }
    return true;
  }
  int field() const { return field_; }
  int wire() const { return wire_; }
  // a scalar field (varint or fixed width)
  uint64_t value() const {
    if (wire_ == 2) {
      throw std::runtime_error("protowire: field " + std::to_string(field_) + " is length-delimited where a scalar was expected");
    }
    return value_;
  }
  // a string, bytes or nested-message field
  const std::string& bytes() const {
    if (wire_ != 2) {
      throw std::runtime_error("protowire: field " + std::to_string(field_) + " is a scalar where a length-delimited value was expected");
    }
    return bytes_;
  }
  // One occurrence of a repeated integer field: a single value, or a packed run of them (what a
  // proto3 writer, or a proto2 writer with [packed = true], emits for the same schema).
  template <typename F>
  void eachValue(F&& f) const {
    if (wire_ != 2) {
      f(value_);
      return;
    }
    Reader packed(bytes_);
    while (packed.pos_ < packed.s_.size()) {
      f(packed.raw());
    }
  }

 private:
  uint64_t raw() {
    uint64_t v = 0;
    for (int shift = 0; shift < 70; shift += 7) {
      if (pos_ >= s_.size()) {
        throw std::runtime_error("protowire: truncated varint");
      }
      unsigned char c = static_cast<unsigned char>(s_[pos_++]);
      if (shift < 64) {
        v |= static_cast<uint64_t>(c & 0x7f) << shift;
      }
      if (!(c & 0x80)) {
        return v;
      }
    }
    throw std::runtime_error("protowire: varint longer than ten bytes");
  }
  const std::string& s_;
  size_t pos_ = 0;
  int field_ = 0, wire_ = 0;
  uint64_t value_ = 0;
  std::string bytes_;
};

} // namespace protowire
} // namespace tc
