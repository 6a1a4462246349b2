#include "json.h"

#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <sstream>
#include <stdexcept>

#include "Logger.h"

extern Logger logger;

namespace tkjson {

const Value *Value::find(const std::string &key) const
{
    if (kind != Object) return nullptr;
    for (auto &m : members)
        if (m.first == key) return &m.second;
    return nullptr;
}

namespace {
struct Parser {
    const std::string &s;
    size_t i = 0;
    explicit Parser(const std::string &text) : s(text) {}
    [[noreturn]] void fail(const char *what)
    {
        throw std::runtime_error("json: " + std::string(what) + " at byte " + std::to_string(i));
    }
    void ws()
    {
        while (i < s.size() && (s[i] == ' ' || s[i] == '\t' || s[i] == '\n' || s[i] == '\r')) ++i;
    }
    std::string str()
    {
        if (s[i] != '"') fail("expected string");
        ++i;
        std::string out;
        while (i < s.size() && s[i] != '"') {
            if (s[i] == '\\') {
                if (++i >= s.size()) fail("bad escape");
                switch (s[i]) {
                    case 'n': out += '\n'; break;
                    case 't': out += '\t'; break;
                    case 'r': out += '\r'; break;
                    case 'b': out += '\b'; break;
                    case 'f': out += '\f'; break;
                    case 'u': {
                        if (i + 4 >= s.size()) fail("bad \\u escape");
                        unsigned cp = (unsigned)strtoul(s.substr(i + 1, 4).c_str(), nullptr, 16);
                        out += (cp < 0x80) ? (char)cp : '?';
                        i += 4;
                        break;
                    }
                    default: out += s[i];
                }
                ++i;
            } else {
                out += s[i++];
            }
        }
        if (i >= s.size()) fail("unterminated string");
        ++i;
        return out;
    }
    Value value()
    {
        ws();
        if (i >= s.size()) fail("unexpected end");
        Value v;
        const char c = s[i];
        if (c == '{') {
            v.kind = Value::Object;
            ++i;
            ws();
            if (i < s.size() && s[i] == '}') { ++i; return v; }
            for (;;) {
                ws();
                std::string key = str();
                ws();
                if (i >= s.size() || s[i] != ':') fail("expected ':'");
                ++i;
                v.members.emplace_back(std::move(key), value());
                ws();
                if (i < s.size() && s[i] == ',') { ++i; continue; }
                if (i < s.size() && s[i] == '}') { ++i; break; }
                fail("expected ',' or '}'");
            }
        } else if (c == '[') {
            v.kind = Value::Array;
            ++i;
            ws();
            if (i < s.size() && s[i] == ']') { ++i; return v; }
            for (;;) {
                v.items.push_back(value());
                ws();
                if (i < s.size() && s[i] == ',') { ++i; continue; }
                if (i < s.size() && s[i] == ']') { ++i; break; }
                fail("expected ',' or ']'");
            }
        } else if (c == '"') {
            v.kind = Value::String;
            v.text = str();
        } else if (s.compare(i, 4, "true") == 0) {
            v.kind = Value::Bool; v.boolean = true; i += 4;
        } else if (s.compare(i, 5, "false") == 0) {
            v.kind = Value::Bool; i += 5;
        } else if (s.compare(i, 4, "null") == 0) {
            i += 4;
        } else {
            const size_t b = i;
            while (i < s.size() && (isdigit((unsigned char)s[i]) || s[i] == '-' || s[i] == '+' ||
                                    s[i] == '.' || s[i] == 'e' || s[i] == 'E'))
                ++i;
            if (b == i) fail("unexpected character");
            v.kind = Value::Number;
            v.text = s.substr(b, i - b);
            v.number = strtod(v.text.c_str(), nullptr);
        }
        return v;
    }
};
}  // namespace

Value parse(const std::string &text)
{
    Parser p(text);
    Value v = p.value();
    p.ws();
    if (p.i != text.size()) p.fail("trailing characters");
    return v;
}

}  // namespace tkjson

static tkjson::Value ptr;          // the model's kinfo tree
static tkjson::Value common_ptr;   // kinfo-common

static const tkjson::Value *lookup(const std::string &kernel_name, const std::string &key)
{
    const tkjson::Value *k = ptr.find(kernel_name);
    return k ? k->find(key) : nullptr;
}

int get_kernel_info(const std::string &kernel_name, const std::string &key)
{
    const tkjson::Value *v = lookup(kernel_name, key);
    if (!v || v->kind != tkjson::Value::Number) return JSON_NOT_FOUND;
    return (int)v->number;
}

float fget_kernel_info(const std::string &kernel_name, const std::string &key)
{
    const tkjson::Value *v = lookup(kernel_name, key);
    if (!v || v->kind != tkjson::Value::Number) return JSON_NOT_FOUND;
    return (float)v->number;
}

std::string sget_kernel_info(const std::string &kernel_name, const std::string &key)
{
    const tkjson::Value *v = lookup(kernel_name, key);
    if (!v) return "";
    return v->text;
}

static std::string slurp(const std::string &filename)
{
    std::ifstream file(filename);
    if (!file.is_open()) {
        std::cerr << "Error: file not found: " << filename << std::endl;
        exit(1);
    }
    std::stringstream ss;
    ss << file.rdbuf();
    return ss.str();
}

void read_json_text(const std::string &text) { ptr = tkjson::parse(text); }

void read_json(const std::string &filename)
{
    read_json_text(slurp(filename));
    logger.INFO("Read json file: " + filename);
}

void add_kernel_info(const std::string &kernel_name, const std::string &key, const int value)
{
    if (ptr.kind != tkjson::Value::Object) ptr.kind = tkjson::Value::Object;
    tkjson::Value *k = const_cast<tkjson::Value *>(ptr.find(kernel_name));
    if (!k) {
        ptr.members.emplace_back(kernel_name, tkjson::Value());
        k = &ptr.members.back().second;
        k->kind = tkjson::Value::Object;
    }
    tkjson::Value num;
    num.kind = tkjson::Value::Number;
    num.number = value;
    num.text = std::to_string(value);
    tkjson::Value *slot = const_cast<tkjson::Value *>(k->find(key));
    if (slot) *slot = num;
    else k->members.emplace_back(key, num);
}

static void write_value(std::ostream &os, const tkjson::Value &v, int indent)
{
    const std::string pad(indent, ' ');
    switch (v.kind) {
        case tkjson::Value::Object: {
            os << "{\n";
            for (size_t n = 0; n < v.members.size(); ++n) {
                os << pad << "    \"" << v.members[n].first << "\": ";
                write_value(os, v.members[n].second, indent + 4);
                os << (n + 1 < v.members.size() ? ",\n" : "\n");
            }
            os << pad << "}";
            break;
        }
        case tkjson::Value::Array: {
            os << "[";
            for (size_t n = 0; n < v.items.size(); ++n) {
                write_value(os, v.items[n], indent + 4);
                if (n + 1 < v.items.size()) os << ", ";
            }
            os << "]";
            break;
        }
        case tkjson::Value::String: os << '"' << v.text << '"'; break;
        case tkjson::Value::Number: os << v.text; break;
        case tkjson::Value::Bool: os << (v.boolean ? "true" : "false"); break;
        default: os << "null";
    }
}

void build_json(const std::string &filename)
{
    std::ofstream file(filename);
    if (!file.is_open()) {
        std::cerr << "Error: file not found" << std::endl;
        exit(1);
    }
    write_value(file, ptr, 0);
    file << "\n";
}

void read_common_json_text(const std::string &text) { common_ptr = tkjson::parse(text); }

void read_common_json(const std::string &filename)
{
    read_common_json_text(slurp(filename));
    logger.INFO("Read json file: " + filename);
}

long long geti(int count, const char *keys...)
{
    va_list args;
    va_start(args, keys);
    const tkjson::Value *tmp = &common_ptr;
    std::vector<const char *> key_list;
    for (int i = 0; i < count; i++) {
        const char *key = (!i) ? keys : va_arg(args, const char *);
        key_list.push_back(key);
        const tkjson::Value *next = tmp->find(key);
        if (!next) {
            printf("key chain: ");
            for (auto k : key_list) printf("%s -> ", k);
            printf("END, not found!\n");
            va_end(args);
            exit(1);
        }
        tmp = next;
    }
    va_end(args);
    return (long long)tmp->number;
}
