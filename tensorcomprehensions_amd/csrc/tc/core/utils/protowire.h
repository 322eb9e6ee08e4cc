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
    if (wire_ == 0) {
      value_ = raw();
    } else if (wire_ == 2) {
      uint64_t n = raw();
      if (pos_ + n > s_.size()) {
        throw std::runtime_error("protowire: truncated length-delimited field");
      }
      bytes_ = s_.substr(pos_, n);
      pos_ += n;
    } else if (wire_ == 1) {
      value_ = 0;
      for (int i = 0; i < 8; ++i) {
        value_ |= static_cast<uint64_t>(static_cast<unsigned char>(s_.at(pos_ + i))) << (8 * i);
      }
      pos_ += 8;
    } else if (wire_ == 5) {
      pos_ += 4;
    } else {
      throw std::runtime_error("protowire: unsupported wire type");
    }
    return true;
  }
  int field() const { return field_; }
  int wire() const { return wire_; }
  uint64_t value() const { return value_; }
  const std::string& bytes() const { return bytes_; }

 private:
  uint64_t raw() {
    uint64_t v = 0;
    int shift = 0;
    for (;;) {
      if (pos_ >= s_.size()) {
        throw std::runtime_error("protowire: truncated varint");
      }
      unsigned char c = static_cast<unsigned char>(s_[pos_++]);
      v |= static_cast<uint64_t>(c & 0x7f) << shift;
      if (!(c & 0x80)) {
        return v;
      }
      shift += 7;
    }
  }
  const std::string& s_;
  size_t pos_ = 0;
  int field_ = 0, wire_ = 0;
  uint64_t value_ = 0;
  std::string bytes_;
};

} // namespace protowire
} // namespace tc
