// Json.cpp — recursive-descent reader behind Json.h.
#include "Json.h"

#include <cctype>
#include <cmath>
#include <cstdlib>
#include <fstream>
#include <sstream>
#include <stdexcept>

namespace json {

static const char* kTypeName[] = {"null", "a boolean", "a number", "a string", "an array", "an object"};

double Value::asDouble() const
{
    if (_type == Number) return _number;
    if (_type == Bool) return _bool ? 1.0 : 0.0;
    if (_type == Null) return 0.0;
    throw std::runtime_error(std::string("json: expected a number, found ") + kTypeName[_type]);
}

int64_t Value::asInt() const { return (int64_t)asDouble(); }

bool Value::asBool() const
{
    if (_type == Bool) return _bool;
    if (_type == Number) return _number != 0.0;
    if (_type == Null) return false;
    throw std::runtime_error(std::string("json: expected a boolean, found ") + kTypeName[_type]);
}

const std::string& Value::asString() const
{
    if (_type != String) throw std::runtime_error(std::string("json: expected a string, found ") + kTypeName[_type]);
    return _string;
}

const Value* Value::find(const std::string& key) const
{
    for (auto& m : _members)
        if (m.first == key) return &m.second;
    return nullptr;
}

std::string lower(const std::string& s)
{
    std::string r(s);
    for (auto& c : r) c = (char)std::tolower((unsigned char)c);
    return r;
}

class Parser {
    const std::string& _s;
    size_t _p;

    [[noreturn]] void fail(const std::string& what) const
    {
        size_t line = 1, col = 1;
        for (size_t i = 0; i < _p && i < _s.size(); i++) {
            if (_s[i] == '\n') {
                line++;
                col = 1;
            } else
                col++;
        }
        std::ostringstream o;
        o << "line " << line << ", column " << col << ": " << what;
        throw std::runtime_error(o.str());
    }

    void skip()
    {
        for (;;) {
            while (_p < _s.size() && std::isspace((unsigned char)_s[_p])) _p++;
            if (_p + 1 < _s.size() && _s[_p] == '/' && _s[_p + 1] == '/') {
                while (_p < _s.size() && _s[_p] != '\n') _p++;
            } else if (_p + 1 < _s.size() && _s[_p] == '/' && _s[_p + 1] == '*') {
                size_t e = _s.find("*/", _p + 2);
                if (e == std::string::npos) fail("comment without end");
                _p = e + 2;
            } else
                return;
        }
    }

    static void appendUtf8(std::string& out, uint32_t cp)
    {
        if (cp < 0x80)
            out += (char)cp;
        else if (cp < 0x800) {
            out += (char)(0xC0 | (cp >> 6));
            out += (char)(0x80 | (cp & 0x3F));
        } else if (cp < 0x10000) {
            out += (char)(0xE0 | (cp >> 12));
            out += (char)(0x80 | ((cp >> 6) & 0x3F));
            out += (char)(0x80 | (cp & 0x3F));
        } else {
            out += (char)(0xF0 | (cp >> 18));
            out += (char)(0x80 | ((cp >> 12) & 0x3F));
            out += (char)(0x80 | ((cp >> 6) & 0x3F));
            out += (char)(0x80 | (cp & 0x3F));
        }
    }

    uint32_t hex4()
    {
        if (_p + 4 > _s.size()) fail("short \\u escape");
        uint32_t v = 0;
        for (int i = 0; i < 4; i++) {
            char c = _s[_p++];
            v <<= 4;
            if (c >= '0' && c <= '9')
                v |= (uint32_t)(c - '0');
            else if (c >= 'a' && c <= 'f')
                v |= (uint32_t)(c - 'a' + 10);
            else if (c >= 'A' && c <= 'F')
                v |= (uint32_t)(c - 'A' + 10);
            else
                fail("bad \\u escape");
        }
        return v;
    }

    std::string string()
    {
        if (_s[_p] != '"') fail("expected '\"'");
        _p++;
        std::string out;
        while (true) {
            if (_p >= _s.size()) fail("string without end");
            char c = _s[_p++];
            if (c == '"') return out;
            if (c != '\\') {
                out += c;
                continue;
            }
            if (_p >= _s.size()) fail("string without end");
            char e = _s[_p++];
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
                uint32_t cp = hex4();
                if (cp >= 0xD800 && cp < 0xDC00 && _p + 1 < _s.size() && _s[_p] == '\\' && _s[_p + 1] == 'u') {
                    _p += 2;
                    uint32_t lo = hex4();
                    cp = 0x10000 + ((cp - 0xD800) << 10) + (lo - 0xDC00);
                }
                appendUtf8(out, cp);
                break;
            }
            default: fail("unknown escape in string");
            }
        }
    }

    void value(Value& v, int depth)
    {
        if (depth > 256) fail("nesting too deep");
        skip();
        if (_p >= _s.size()) fail("value expected, found the end of the text");
        char c = _s[_p];
        if (c == '{') {
            _p++;
            v._type = Value::Object;
            skip();
            if (_p < _s.size() && _s[_p] == '}') {
                _p++;
                return;
            }
            while (true) {
                skip();
                if (_p >= _s.size() || _s[_p] != '"') fail("member name expected");
                std::string key = string();
                skip();
                if (_p >= _s.size() || _s[_p] != ':') fail("':' expected after member name");
                _p++;
                v._members.emplace_back(std::move(key), Value());
                value(v._members.back().second, depth + 1);
                skip();
                if (_p < _s.size() && _s[_p] == ',') {
                    _p++;
                    continue;
                }
                if (_p < _s.size() && _s[_p] == '}') {
                    _p++;
                    return;
                }
                fail("',' or '}' expected in object");
            }
        } else if (c == '[') {
            _p++;
            v._type = Value::Array;
            skip();
            if (_p < _s.size() && _s[_p] == ']') {
                _p++;
                return;
            }
            while (true) {
                v._items.emplace_back();
                value(v._items.back(), depth + 1);
                skip();
                if (_p < _s.size() && _s[_p] == ',') {
                    _p++;
                    continue;
                }
                if (_p < _s.size() && _s[_p] == ']') {
                    _p++;
                    return;
                }
                fail("',' or ']' expected in array");
            }
        } else if (c == '"') {
            v._type = Value::String;
            v._string = string();
        } else if (_s.compare(_p, 4, "true") == 0) {
            v._type = Value::Bool;
            v._bool = true;
            _p += 4;
        } else if (_s.compare(_p, 5, "false") == 0) {
            v._type = Value::Bool;
            v._bool = false;
            _p += 5;
        } else if (_s.compare(_p, 4, "null") == 0) {
            v._type = Value::Null;
            _p += 4;
        } else if (c == '-' || c == '+' || (c >= '0' && c <= '9') || c == '.') {
            const char* b = _s.c_str() + _p;
            char* e = nullptr;
            double d = std::strtod(b, &e);
            if (e == b) fail("bad number");
            _p += (size_t)(e - b);
            v._type = Value::Number;
            v._number = d;
        } else
            fail(std::string("unexpected character '") + c + "'");
    }

public:
    explicit Parser(const std::string& s) : _s(s), _p(0) {}

    void document(Value& root)
    {
        value(root, 0);
        skip();
        if (_p != _s.size()) fail("text after the end of the document");
    }
};

bool parse(const std::string& text, Value& root, std::string& error)
{
    root = Value();
    try {
        Parser(text).document(root);
    } catch (std::exception& e) {
        error = e.what();
        return false;
    }
    return true;
}

bool parseFile(const std::string& path, Value& root, std::string& error)
{
    std::ifstream in(path, std::ios::binary);
    if (!in) {
        error = "cannot open " + path;
        return false;
    }
    std::stringstream buf;
    buf << in.rdbuf();
    return parse(buf.str(), root, error);
}

}  // namespace json
