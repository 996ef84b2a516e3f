#include "json_reader.h"

#include "forest.h"

#include <cerrno>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>

namespace tbamd {

namespace {

struct Parser {
  const char *p, *end;

  [[noreturn]] void Fail(const char *what) { throw Error(std::string("JSON: ") + what); }
  void SkipWs() {
    while (p < end && (*p == ' ' || *p == '\n' || *p == '\r' || *p == '\t')) ++p;
  }
  char Peek() {
    SkipWs();
    if (p >= end) Fail("unexpected end of input");
    return *p;
  }
  void Expect(char c) {
    if (Peek() != c) Fail("unexpected character");
    ++p;
  }

  static void AppendUtf8(std::string &out, uint32_t cp) {
    if (cp < 0x80) out += (char)cp;
    else if (cp < 0x800) { out += (char)(0xC0 | (cp >> 6)); out += (char)(0x80 | (cp & 0x3F)); }
    else if (cp < 0x10000) { out += (char)(0xE0 | (cp >> 12)); out += (char)(0x80 | ((cp >> 6) & 0x3F)); out += (char)(0x80 | (cp & 0x3F)); }
    else { out += (char)(0xF0 | (cp >> 18)); out += (char)(0x80 | ((cp >> 12) & 0x3F)); out += (char)(0x80 | ((cp >> 6) & 0x3F)); out += (char)(0x80 | (cp & 0x3F)); }
  }

  uint32_t Hex4() {
    if (end - p < 4) Fail("bad \\u escape");
    uint32_t v = 0;
    for (int i = 0; i < 4; ++i) {
      char c = *p++;
      v <<= 4;
      if (c >= '0' && c <= '9') v |= c - '0';
      else if (c >= 'a' && c <= 'f') v |= c - 'a' + 10;
      else if (c >= 'A' && c <= 'F') v |= c - 'A' + 10;
      else Fail("bad \\u escape");
    }
    return v;
  }

  std::string String() {
    Expect('"');
    std::string out;
    while (true) {
      if (p >= end) Fail("unterminated string");
      char c = *p++;
      if (c == '"') break;
      if (c != '\\') { out += c; continue; }
      if (p >= end) Fail("unterminated escape");
      char e = *p++;
      switch (e) {
      case '"': out += '"'; break;
      case '\\': out += '\\'; break;
      case '/': out += '/'; break;
      case 'b': out += '\b'; break;
      case 'f': out += '\f'; break;
      case 'n': out += '\n'; break;
      case 'r': out += '\r'; break;
      case 't': out += '\t'; break;
      case 'u': {
        uint32_t cp = Hex4();
        if (cp >= 0xD800 && cp < 0xDC00 && end - p >= 6 && p[0] == '\\' && p[1] == 'u') {
          p += 2;
          uint32_t lo = Hex4();
          cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
        }
        AppendUtf8(out, cp);
        break;
      }
      default: Fail("bad escape");
      }
    }
    return out;
  }

  double Number() {
    // strtod needs a terminated buffer; numbers are short, copy them out.
    char buf[64];
    size_t n = 0;
    while (p < end && n + 1 < sizeof(buf) &&
           ((*p >= '0' && *p <= '9') || *p == '-' || *p == '+' || *p == '.' || *p == 'e' || *p == 'E'))
      buf[n++] = *p++;
    buf[n] = 0;
    if (n == 0) Fail("bad number");
    char *stop = nullptr;
    double v = std::strtod(buf, &stop);
    if (stop != buf + n) Fail("bad number");
    return v;
  }

  bool Literal(const char *word) {
    size_t n = std::strlen(word);
    if ((size_t)(end - p) >= n && std::memcmp(p, word, n) == 0) { p += n; return true; }
    return false;
  }

  JsonValue Value(int depth) {
    if (depth > 256) Fail("nesting too deep");
    JsonValue v;
    char c = Peek();
    if (c == '{') {
      ++p;
      v.kind = JsonValue::Kind::kObject;
      if (Peek() == '}') { ++p; return v; }
      while (true) {
        SkipWs();
        std::string key = String();
        Expect(':');
        v.object.emplace_back(std::move(key), Value(depth + 1));
        char d = Peek();
        ++p;
        if (d == '}') break;
        if (d != ',') Fail("expected , or }");
      }
    } else if (c == '[') {
      ++p;
      v.kind = JsonValue::Kind::kNumberArray; // until a non-number shows up
      if (Peek() == ']') { ++p; return v; }
      while (true) {
        char f = Peek();
        bool isNum = (f == '-' || (f >= '0' && f <= '9'));
        if (isNum && v.kind == JsonValue::Kind::kNumberArray) {
          v.numbers.push_back(Number());
        } else {
          if (v.kind == JsonValue::Kind::kNumberArray) {
            v.kind = JsonValue::Kind::kArray;
            for (double d : v.numbers) {
              JsonValue e;
              e.kind = JsonValue::Kind::kNumber;
              e.number = d;
              v.array.push_back(std::move(e));
            }
            v.numbers.clear();
          }
          v.array.push_back(Value(depth + 1));
        }
        char d = Peek();
        ++p;
        if (d == ']') break;
        if (d != ',') Fail("expected , or ]");
      }
    } else if (c == '"') {
      v.kind = JsonValue::Kind::kString;
      v.str = String();
    } else if (c == 't' || c == 'f') {
      v.kind = JsonValue::Kind::kBool;
      if (Literal("true")) v.boolean = true;
      else if (Literal("false")) v.boolean = false;
      else Fail("bad literal");
    } else if (c == 'n') {
      if (!Literal("null")) Fail("bad literal");
    } else {
      v.kind = JsonValue::Kind::kNumber;
      v.number = Number();
    }
    return v;
  }
};

} // namespace

bool JsonValue::Has(const std::string &key) const {
  for (auto &kv : object)
    if (kv.first == key) return true;
  return false;
}

const JsonValue &JsonValue::operator[](const std::string &key) const {
  for (auto &kv : object)
    if (kv.first == key) return kv.second;
  throw Error("JSON: missing key \"" + key + "\"");
}

size_t JsonValue::Size() const {
  switch (kind) {
  case Kind::kArray: return array.size();
  case Kind::kNumberArray: return numbers.size();
  case Kind::kObject: return object.size();
  default: return 0;
  }
}

std::vector<double> JsonValue::AsNumbers() const {
  if (kind == Kind::kNumberArray) return numbers;
  if (kind != Kind::kArray) throw Error("JSON: expected an array");
  std::vector<double> out;
  for (auto &e : array) {
    if (e.kind == Kind::kNumber) out.push_back(e.number);
    else if (e.kind == Kind::kBool) out.push_back(e.boolean ? 1.0 : 0.0);
    else throw Error("JSON: expected a numeric array");
  }
  return out;
}

const std::string &JsonValue::AsString() const {
  if (kind != Kind::kString) throw Error("JSON: expected a string");
  return str;
}

double JsonValue::AsNumber() const {
  if (kind != Kind::kNumber) throw Error("JSON: expected a number");
  return number;
}

JsonValue ParseJson(const char *begin, const char *end) {
  Parser parser{begin, end};
  JsonValue v = parser.Value(0);
  parser.SkipWs();
  if (parser.p != end) throw Error("JSON: trailing characters");
  return v;
}

std::string ReadFile(const std::string &path) {
  std::ifstream in(path, std::ios::binary);
  if (!in) throw Error("cannot open " + path);
  std::ostringstream ss;
  ss << in.rdbuf();
  return ss.str();
}

JsonValue ParseJsonFile(const std::string &path) {
  std::string text = ReadFile(path);
  return ParseJson(text.data(), text.data() + text.size());
}

} // namespace tbamd
