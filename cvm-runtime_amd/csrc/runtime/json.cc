#include "json.h"

#include <cctype>
#include <cstdlib>

namespace cvmrt {
namespace {

class Parser {
 public:
  explicit Parser(const std::string& t) : t_(t), p_(0) {}

  Json Document() {
    Json v = Value(0);
    Skip();
    CVM_CHECK(p_ == t_.size()) << "json: trailing characters at offset " << p_;
    return v;
  }

 private:
  void Skip() {
    while (p_ < t_.size() && std::isspace(static_cast<unsigned char>(t_[p_]))) ++p_;
  }
  char Peek() {
    Skip();
    CVM_CHECK(p_ < t_.size()) << "json: unexpected end of input";
    return t_[p_];
  }
  void Expect(char c) {
    CVM_CHECK(Peek() == c) << "json: expected '" << c << "' at offset " << p_ << " but found '" << t_[p_] << "'";
    ++p_;
  }

  std::string String() {
    Expect('"');
    std::string out;
    while (true) {
      CVM_CHECK(p_ < t_.size()) << "json: unterminated string";
      char c = t_[p_++];
      if (c == '"') break;
      if (c == '\\') {
        CVM_CHECK(p_ < t_.size()) << "json: unterminated escape";
        char e = t_[p_++];
        switch (e) {
          case 'n': out.push_back('\n'); break;
          case 't': out.push_back('\t'); break;
          case 'r': out.push_back('\r'); break;
          case 'b': out.push_back('\b'); break;
          case 'f': out.push_back('\f'); break;
          case '/': out.push_back('/'); break;
          case '\\': out.push_back('\\'); break;
          case '"': out.push_back('"'); break;
          case 'u': {
            CVM_CHECK(p_ + 4 <= t_.size()) << "json: bad \\u escape";
            unsigned cp = static_cast<unsigned>(std::strtoul(t_.substr(p_, 4).c_str(), nullptr, 16));
            p_ += 4;
            if (cp < 0x80) out.push_back(static_cast<char>(cp));
            else if (cp < 0x800) { out.push_back(static_cast<char>(0xC0 | (cp >> 6))); out.push_back(static_cast<char>(0x80 | (cp & 0x3F))); }
            else { out.push_back(static_cast<char>(0xE0 | (cp >> 12))); out.push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F))); out.push_back(static_cast<char>(0x80 | (cp & 0x3F))); }
            break;
          }
          default: CVM_FATAL() << "json: unknown escape \\" << e;
        }
      } else {
        out.push_back(c);
      }
    }
    return out;
  }

  Json Number() {
    size_t start = p_;
    if (t_[p_] == '-' || t_[p_] == '+') ++p_;
    bool integral = true;
    while (p_ < t_.size()) {
      char c = t_[p_];
      if (std::isdigit(static_cast<unsigned char>(c))) { ++p_; continue; }
      if (c == '.' || c == 'e' || c == 'E' || c == '-' || c == '+') { integral = false; ++p_; continue; }
      break;
    }
    CVM_CHECK(p_ > start) << "json: bad number at offset " << start;
    Json v;
    std::string tok = t_.substr(start, p_ - start);
    if (integral) {
      v.kind = Json::kInt;
      v.i = std::strtoll(tok.c_str(), nullptr, 10);
      v.d = static_cast<double>(v.i);
    } else {
      v.kind = Json::kDouble;
      v.d = std::strtod(tok.c_str(), nullptr);
      v.i = static_cast<int64_t>(v.d);
    }
    return v;
  }

  Json Value(int depth) {
    CVM_CHECK(depth < 64) << "json: nesting too deep";
    char c = Peek();
    Json v;
    if (c == '{') {
      ++p_;
      v.kind = Json::kObject;
      if (Peek() == '}') { ++p_; return v; }
      while (true) {
        std::string key = String();
        Expect(':');
        v.obj.emplace_back(std::move(key), Value(depth + 1));
        char n = Peek();
        ++p_;
        if (n == '}') break;
        CVM_CHECK(n == ',') << "json: expected ',' or '}' at offset " << p_ - 1;
      }
    } else if (c == '[') {
      ++p_;
      v.kind = Json::kArray;
      if (Peek() == ']') { ++p_; return v; }
      while (true) {
        v.arr.push_back(Value(depth + 1));
        char n = Peek();
        ++p_;
        if (n == ']') break;
        CVM_CHECK(n == ',') << "json: expected ',' or ']' at offset " << p_ - 1;
      }
    } else if (c == '"') {
      v.kind = Json::kString;
      v.s = String();
    } else if (t_.compare(p_, 4, "true") == 0) {
      v.kind = Json::kBool; v.b = true; p_ += 4;
    } else if (t_.compare(p_, 5, "false") == 0) {
      v.kind = Json::kBool; v.b = false; p_ += 5;
    } else if (t_.compare(p_, 4, "null") == 0) {
      p_ += 4;
    } else {
      v = Number();
    }
    return v;
  }

  const std::string& t_;
  size_t p_;
};

}  // namespace

Json Json::Parse(const std::string& text) { return Parser(text).Document(); }

}  // namespace cvmrt
