// json.h -- kinfo configuration lookups (src/json.h of the reference).
//
// Same free functions and the same "missing key" convention (JSON_NOT_FOUND =
// -INT16_MAX).  The reference parses with Boost.PropertyTree; this is a small
// self-contained reader for the subset the kinfo files use (objects, numbers,
// strings, arrays, true/false/null).
#pragma once
#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

const int JSON_NOT_FOUND = -INT16_MAX;

namespace tkjson {
struct Value {
    enum Kind { Null, Bool, Number, String, Array, Object } kind = Null;
    double number = 0.0;
    bool boolean = false;
    std::string text;                                  // String, and the literal of a Number
    std::vector<Value> items;                          // Array
    std::vector<std::pair<std::string, Value>> members;  // Object, in file order
    const Value *find(const std::string &key) const;
};
// throws std::runtime_error with the byte offset on malformed input
Value parse(const std::string &text);
}  // namespace tkjson

void read_json(const std::string &filename);          // exits(1) if the file is missing
void read_json_text(const std::string &text);         // same, from memory
float fget_kernel_info(const std::string &kernel_name, const std::string &key);
int get_kernel_info(const std::string &kernel_name, const std::string &key);
void add_kernel_info(const std::string &kernel_name, const std::string &key, const int value);
void build_json(const std::string &filename);
std::string sget_kernel_info(const std::string &kernel_name, const std::string &key);

// kinfo-common.json: geti(n, "k1", ..., "kn") walks n keys; exits(1) on a missing key
long long geti(int count, const char *keys...);
void read_common_json(const std::string &filename);
void read_common_json_text(const std::string &text);
