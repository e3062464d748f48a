// Minimal JSON document reader/writer for the three inputs of the token loop:
// vocab.json (array of strings), tokenised stories (array of arrays of strings)
// and the model.bin header (nested objects with "shape"/"dtype").  The
// reference parses these with its vendored cJSON (load_model.cu:224, 349;
// main.cu:76); this reader accepts the same documents and keeps object keys
// in file order.
#pragma once

#include <memory>
#include <string>
#include <utility>
#include <vector>

namespace mll {

struct Json {
    enum Type { Null, Bool, Number, String, Array, Object };
    Type type = Null;
    bool b = false;
    double num = 0;
    std::string str;
    std::vector<Json> arr;
    std::vector<std::pair<std::string, Json>> obj; // file order

    bool isArray() const { return type == Array; }
    bool isObject() const { return type == Object; }
    bool isString() const { return type == String; }
    bool isNumber() const { return type == Number; }
    // First member with that key (cJSON_GetObjectItem semantics, but case-sensitive), or nullptr.
    const Json* get(const std::string& key) const;
    int asInt() const { return (int)num; }
};

// Parses a complete document.  On failure returns false and describes the error
// (with byte offset) in err.  Nesting deeper than 256 levels is rejected.
bool parseJson(const char* text, size_t len, Json& out, std::string& err);

// Compact serialisation (no whitespace); strings escaped per RFC 8259.
std::string dumpJson(const Json& j);

Json jsonNumber(double v);
Json jsonString(const std::string& s);
Json jsonIntArray(const std::vector<int>& v);

} // namespace mll
