// JSON schema -> GBNF text, behind retro_grammar_from_json_schema (reference
// crates/retrograd-ffi/runtime/src/retro_grammar.cpp:36-47, which calls json_schema_to_grammar of llama.cpp's
// common/, absent from the reference checkout). Written for this library; the subset of JSON Schema that
// structured-output callers use, and a refusal that names the keyword for the rest:
//
//   type        object | array | string | number | integer | boolean | null, or a list of those
//   object      properties (in the schema's order; those in `required` must appear, the others may be left out),
//               additionalProperties (true or a schema: further members after the declared ones; absent or false:
//               none - but an object schema without properties takes any object)
//   array       items, prefixItems (a tuple), minItems, maxItems
//   string      minLength, maxLength; enum / const of any JSON values; `format` is read as documentation
//   anyOf / oneOf (alternatives), $ref to #/definitions/NAME or #/$defs/NAME (may be recursive), true / {} (any value)
//   title, description, default, examples, $schema, $id are ignored
//
// Not built (an error says so): pattern, minimum / maximum and their exclusive forms, multipleOf, allOf, not,
// if / then / else, patternProperties, propertyNames, uniqueItems, contains, remote $ref.
//
// The text between tokens is at most one space, so that a model cannot wander off into white space.
#pragma once

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <map>
#include <memory>
#include <set>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace retro {

struct JsonValue {
    enum Kind { NUL, BOOL, NUMBER, STRING, ARRAY, OBJECT } kind = NUL;
    bool b = false;
    double num = 0.0;
    std::string text;                                         // STRING: the decoded text; NUMBER: as written
    std::vector<JsonValue> items;
    std::vector<std::pair<std::string, JsonValue>> members;   // in the order written

    const JsonValue * get(const std::string & key) const {
        for (const auto & m : members) if (m.first == key) return &m.second;
        return nullptr;
    }
};

class JsonParser {
public:
    static JsonValue parse(const std::string & s) {
        JsonParser p(s);
        p.ws();
        JsonValue v = p.value(0);
        p.ws();
        if (p.at_ != s.size()) p.fail("text after the JSON value");
        return v;
    }

private:
    explicit JsonParser(const std::string & s) : s_(s) {}
    const std::string & s_;
    size_t at_ = 0;

    [[noreturn]] void fail(const std::string & what) const {
        throw std::runtime_error("invalid JSON at offset " + std::to_string(at_) + ": " + what);
    }
    char peek() const { return at_ < s_.size() ? s_[at_] : '\0'; }
    void ws() { while (at_ < s_.size() && (s_[at_] == ' ' || s_[at_] == '\t' || s_[at_] == '\n' || s_[at_] == '\r')) ++at_; }
    bool take(const char * word) {
        const size_t n = std::char_traits<char>::length(word);
        if (s_.compare(at_, n, word) != 0) return false;
        at_ += n;
        return true;
    }
    static void utf8(uint32_t cp, std::string & o) {
        if (cp < 0x80) o += (char)cp;
        else if (cp < 0x800) { o += (char)(0xc0 | (cp >> 6)); o += (char)(0x80 | (cp & 0x3f)); }
        else if (cp < 0x10000) { o += (char)(0xe0 | (cp >> 12)); o += (char)(0x80 | ((cp >> 6) & 0x3f)); o += (char)(0x80 | (cp & 0x3f)); }
        else { o += (char)(0xf0 | (cp >> 18)); o += (char)(0x80 | ((cp >> 12) & 0x3f)); o += (char)(0x80 | ((cp >> 6) & 0x3f)); o += (char)(0x80 | (cp & 0x3f)); }
    }
    uint32_t hex4() {
        uint32_t v = 0;
        for (int i = 0; i < 4; ++i) {
            const char c = peek();
            int d;
            if (c >= '0' && c <= '9') d = c - '0';
            else if (c >= 'a' && c <= 'f') d = c - 'a' + 10;
            else if (c >= 'A' && c <= 'F') d = c - 'A' + 10;
            else fail("a hexadecimal digit is expected");
            v = v * 16 + (uint32_t)d;
            ++at_;
        }
        return v;
    }
    std::string string() {
        if (peek() != '"') fail("a string is expected");
        ++at_;
        std::string o;
        for (;;) {
            if (at_ >= s_.size()) fail("unterminated string");
            const unsigned char c = (unsigned char)s_[at_++];
            if (c == '"') return o;
            if (c < 0x20) fail("a control character inside a string");
            if (c != '\\') { o += (char)c; continue; }
            const char e = peek();
            ++at_;
            switch (e) {
                case '"': o += '"'; break;
                case '\\': o += '\\'; break;
                case '/': o += '/'; break;
                case 'b': o += '\b'; break;
                case 'f': o += '\f'; break;
                case 'n': o += '\n'; break;
                case 'r': o += '\r'; break;
                case 't': o += '\t'; break;
                case 'u': {
                    uint32_t cp = hex4();
                    if (cp >= 0xd800 && cp < 0xdc00 && peek() == '\\' && at_ + 1 < s_.size() && s_[at_ + 1] == 'u') {
                        at_ += 2;
                        const uint32_t lo = hex4();
                        if (lo >= 0xdc00 && lo < 0xe000) cp = 0x10000 + ((cp - 0xd800) << 10) + (lo - 0xdc00);
                        else fail("a low surrogate is expected");
                    }
                    utf8(cp, o);
                    break;
                }
                default: fail("unknown escape");
            }
        }
    }
    JsonValue value(int depth) {
        if (depth > 200) fail("nested too deeply");
        JsonValue v;
        const char c = peek();
        if (c == '{') {
            ++at_;
            v.kind = JsonValue::OBJECT;
            ws();
            if (peek() == '}') { ++at_; return v; }
            for (;;) {
                ws();
                std::string key = string();
                ws();
                if (peek() != ':') fail("':' is expected");
                ++at_;
                ws();
                v.members.emplace_back(std::move(key), value(depth + 1));
                ws();
                if (peek() == ',') { ++at_; continue; }
                if (peek() == '}') { ++at_; return v; }
                fail("',' or '}' is expected");
            }
        }
        if (c == '[') {
            ++at_;
            v.kind = JsonValue::ARRAY;
            ws();
            if (peek() == ']') { ++at_; return v; }
            for (;;) {
                ws();
                v.items.push_back(value(depth + 1));
                ws();
                if (peek() == ',') { ++at_; continue; }
                if (peek() == ']') { ++at_; return v; }
                fail("',' or ']' is expected");
            }
        }
        if (c == '"') { v.kind = JsonValue::STRING; v.text = string(); return v; }
        if (take("true")) { v.kind = JsonValue::BOOL; v.b = true; return v; }
        if (take("false")) { v.kind = JsonValue::BOOL; return v; }
        if (take("null")) return v;
        const size_t from = at_;
        if (peek() == '-') ++at_;
        if (peek() == '0') ++at_;
        else if (peek() >= '1' && peek() <= '9') while (peek() >= '0' && peek() <= '9') ++at_;
        else fail("a value is expected");
        if (peek() == '.') {
            ++at_;
            if (!(peek() >= '0' && peek() <= '9')) fail("a digit is expected");
            while (peek() >= '0' && peek() <= '9') ++at_;
        }
        if (peek() == 'e' || peek() == 'E') {
            ++at_;
            if (peek() == '+' || peek() == '-') ++at_;
            if (!(peek() >= '0' && peek() <= '9')) fail("a digit is expected");
            while (peek() >= '0' && peek() <= '9') ++at_;
        }
        v.kind = JsonValue::NUMBER;
        v.text = s_.substr(from, at_ - from);
        v.num = std::stod(v.text);
        return v;
    }
};

// A JSON value written out compactly, as the text a constant of a schema must be matched by.
inline void json_text(const JsonValue & v, std::string & o) {
    switch (v.kind) {
        case JsonValue::NUL: o += "null"; return;
        case JsonValue::BOOL: o += v.b ? "true" : "false"; return;
        case JsonValue::NUMBER: o += v.text; return;
        case JsonValue::STRING: {
            o += '"';
            for (unsigned char c : v.text) {
                if (c == '"') o += "\\\"";
                else if (c == '\\') o += "\\\\";
                else if (c == '\n') o += "\\n";
                else if (c == '\r') o += "\\r";
                else if (c == '\t') o += "\\t";
                else if (c < 0x20) { char b[8]; std::snprintf(b, sizeof b, "\\u%04x", c); o += b; }
                else o += (char)c;
            }
            o += '"';
            return;
        }
        case JsonValue::ARRAY:
            o += '[';
            for (size_t i = 0; i < v.items.size(); ++i) { if (i) o += ','; json_text(v.items[i], o); }
            o += ']';
            return;
        case JsonValue::OBJECT:
            o += '{';
            for (size_t i = 0; i < v.members.size(); ++i) {
                if (i) o += ',';
                JsonValue k;
                k.kind = JsonValue::STRING;
                k.text = v.members[i].first;
                json_text(k, o);
                o += ':';
                json_text(v.members[i].second, o);
            }
            o += '}';
            return;
    }
}

class SchemaToGbnf {
public:
    static std::string convert(const std::string & schema_text) {
        const JsonValue schema = JsonParser::parse(schema_text);
        SchemaToGbnf c(schema);
        const std::string root = c.visit(schema, "root");
        std::string out;
        if (root != "root") out += "root ::= " + root + "\n";
        for (const auto & r : c.order_) if (r != "root" || root == "root") out += r + " ::= " + c.rules_[r] + "\n";
        return out;
    }

private:
    explicit SchemaToGbnf(const JsonValue & root) : root_(root) { taken_.insert("root"); }
    const JsonValue & root_;
    std::map<std::string, std::string> rules_;
    std::vector<std::string> order_;
    std::map<std::string, std::string> refs_;            // "#/definitions/x" -> rule name
    std::set<std::string> taken_;

    [[noreturn]] static void refuse(const std::string & keyword) {
        throw std::runtime_error("the JSON schema keyword '" + keyword + "' is not supported by this library's schema converter");
    }

    // A GBNF literal that matches `text` exactly.
    static std::string literal(const std::string & text) {
        std::string o = "\"";
        for (unsigned char c : text) {
            if (c == '"') o += "\\\"";
            else if (c == '\\') o += "\\\\";
            else if (c == '\n') o += "\\n";
            else if (c == '\r') o += "\\r";
            else if (c == '\t') o += "\\t";
            else if (c < 0x20 || c == 0x7f) { char b[8]; std::snprintf(b, sizeof b, "\\x%02X", c); o += b; }
            else o += (char)c;
        }
        return o + "\"";
    }

    std::string define(const std::string & name, const std::string & body) {
        if (!rules_.count(name)) order_.push_back(name);
        rules_[name] = body;
        return name;
    }
    // a rule name nobody uses yet, from a path through the schema
    std::string fresh(const std::string & wish) {
        std::string base;
        for (char c : wish) base += ((c >= 'a' && c <= 'z') || (c >= 'A' && c <= 'Z') || (c >= '0' && c <= '9')) ? c : '-';
        if (base.empty()) base = "rule";
        static const char * const reserved[] = {"space", "char", "string", "number", "integer", "boolean", "null", "value", "object", "array", "member"};
        std::string name = base;
        for (int n = 2;; ++n) {
            bool clash = taken_.count(name) > 0;
            for (const char * r : reserved) clash = clash || name == r;
            if (!clash) break;
            name = base + "-" + std::to_string(n);
        }
        taken_.insert(name);
        return name;
    }

    std::string space() { return define("space", "\" \"?"); }
    std::string chr() {
        return define("char", "[^\"\\\\\\x00-\\x1F] | \"\\\\\" ( [\"\\\\/bfnrt] | \"u\" [0-9a-fA-F]{4} )");
    }
    std::string str() { chr(); space(); return define("string", "\"\\\"\" char* \"\\\"\" space"); }
    std::string integer() { space(); return define("integer", "\"-\"? ( \"0\" | [1-9] [0-9]* ) space"); }
    std::string number() {
        space();
        return define("number", "\"-\"? ( \"0\" | [1-9] [0-9]* ) ( \".\" [0-9]+ )? ( [eE] [-+]? [0-9]+ )? space");
    }
    std::string boolean() { space(); return define("boolean", "( \"true\" | \"false\" ) space"); }
    std::string null() { space(); return define("null", "\"null\" space"); }
    std::string any_value() {
        if (rules_.count("value")) return "value";
        define("value", "");                      // reserves the name: the rules below refer to it
        str(); number(); boolean(); null();
        define("member", "string \":\" space value");
        define("object", "\"{\" space ( member ( \",\" space member )* )? \"}\" space");
        define("array", "\"[\" space ( value ( \",\" space value )* )? \"]\" space");
        return define("value", "object | array | string | number | boolean | null");
    }
    std::string any_object() { any_value(); return "object"; }

    // A JSON string that is none of `taken` (each as it is spelled between the quotes): additionalProperties
    // speaks of the members that properties does not declare. Walks the spellings unit by unit (a character or a
    // whole escape sequence) - as long as the text follows one of them it must leave it before the closing
    // quote. A declared name spelled with other escapes than the plain form (\u0071 for q) is not recognised as
    // that name, and where a declared name continues with a \uXXXX escape no other \u escape is taken there.
    std::string other_key(const std::string & rule, const std::vector<std::string> & taken) {
        chr();
        space();
        struct Node { std::map<std::string, size_t> next; bool ends = false; };
        std::vector<Node> trie(1);
        for (const std::string & t : taken) {
            size_t at = 0;
            for (size_t i = 0; i < t.size();) {
                const unsigned char c = (unsigned char)t[i];
                size_t n = c < 0x80 ? 1 : (c & 0xe0) == 0xc0 ? 2 : (c & 0xf0) == 0xe0 ? 3 : 4;
                if (c == '\\') n = i + 1 < t.size() && t[i + 1] == 'u' ? 6 : 2;
                const std::string unit = t.substr(i, n);
                i += n;
                auto it = trie[at].next.find(unit);
                if (it == trie[at].next.end()) {
                    trie.emplace_back();
                    it = trie[at].next.emplace(unit, trie.size() - 1).first;
                }
                at = it->second;
            }
            trie[at].ends = true;
        }
        std::vector<std::string> names(trie.size());
        for (size_t i = 0; i < trie.size(); ++i) names[i] = fresh(rule + "-other-key-" + std::to_string(i));
        const std::string rest = " char* \"\\\"\" space";
        for (size_t i = 0; i < trie.size(); ++i) {
            // the rest of the key from this node on, closing quote included
            std::vector<std::string> alts;
            if (!trie[i].ends) alts.push_back("\"\\\"\" space");
            std::string apart = "\"\\\\\\x00-\\x1F", letters;
            bool unicode_edge = false;
            for (const auto & e : trie[i].next) {
                alts.push_back(literal(e.first) + " " + names[e.second]);
                if (e.first[0] != '\\') {
                    // the unit's code point, written as an escape inside the class
                    const unsigned char c = (unsigned char)e.first[0];
                    uint32_t cp = e.first.size() == 1 ? c : (uint32_t)(c & (0xff >> (e.first.size() + 1)));
                    for (size_t j = 1; j < e.first.size(); ++j) cp = (cp << 6) | ((unsigned char)e.first[j] & 0x3f);
                    char b[16];
                    if (cp < 0x100) std::snprintf(b, sizeof b, "\\x%02X", cp);
                    else if (cp < 0x10000) std::snprintf(b, sizeof b, "\\u%04X", cp);
                    else std::snprintf(b, sizeof b, "\\U%08X", cp);
                    apart += b;
                } else if (e.first[1] == 'u') {
                    unicode_edge = true;
                } else {
                    letters += e.first[1];
                }
            }
            alts.push_back("[^" + apart + "]" + rest);
            std::string free_letters;
            for (char c : std::string("\"\\/bfnrt")) if (letters.find(c) == std::string::npos) free_letters += (c == '"' || c == '\\') ? std::string("\\") + c : std::string(1, c);
            if (!free_letters.empty()) alts.push_back("\"\\\\\" [" + free_letters + "]" + rest);
            if (!unicode_edge) alts.push_back("\"\\\\u\" [0-9a-fA-F]{4}" + rest);
            std::string body;
            for (size_t k = 0; k < alts.size(); ++k) body += (k ? " | " : "") + alts[k];
            define(names[i], body);
        }
        const std::string key = fresh(rule + "-other-key");
        define(key, "\"\\\"\" " + names[0]);
        return key;
    }

    std::string constant(const JsonValue & v) {
        std::string t;
        json_text(v, t);
        return literal(t) + " " + space();
    }

    const JsonValue & resolve(const std::string & ref) const {
        if (ref.rfind("#/", 0) != 0) refuse("$ref to anything but #/definitions/NAME or #/$defs/NAME");
        const JsonValue * at = &root_;
        size_t from = 2;
        while (from <= ref.size()) {
            size_t to = ref.find('/', from);
            if (to == std::string::npos) to = ref.size();
            std::string key = ref.substr(from, to - from);
            for (size_t p; (p = key.find("~1")) != std::string::npos;) key.replace(p, 2, "/");
            for (size_t p; (p = key.find("~0")) != std::string::npos;) key.replace(p, 2, "~");
            at = at->kind == JsonValue::OBJECT ? at->get(key) : nullptr;
            if (!at) throw std::runtime_error("the JSON schema's $ref '" + ref + "' points at nothing");
            from = to + 1;
        }
        return *at;
    }

    // The name of a rule (or an inline expression) matching `schema`; `name` is the wish for a new rule's name.
    std::string visit(const JsonValue & schema, const std::string & name) {
        if (schema.kind == JsonValue::BOOL) {
            if (!schema.b) refuse("false (a schema nothing satisfies)");
            return any_value();
        }
        if (schema.kind != JsonValue::OBJECT) throw std::runtime_error("a JSON schema must be an object or a boolean");
        static const char * const unsupported[] = {"pattern", "minimum", "maximum", "exclusiveMinimum", "exclusiveMaximum", "multipleOf",
            "allOf", "not", "if", "then", "else", "patternProperties", "propertyNames", "uniqueItems", "contains",
            "minProperties", "maxProperties", "dependentRequired", "dependentSchemas", "unevaluatedProperties"};
        for (const char * k : unsupported) if (schema.get(k)) refuse(k);

        if (const JsonValue * ref = schema.get("$ref")) {
            if (ref->kind != JsonValue::STRING) throw std::runtime_error("$ref must be a string");
            auto it = refs_.find(ref->text);
            if (it != refs_.end()) return it->second;
            const std::string rule = fresh(ref->text.substr(ref->text.rfind('/') + 1));
            refs_[ref->text] = rule;              // before the visit: a definition may refer to itself
            const std::string body = visit(resolve(ref->text), rule);
            if (body != rule) define(rule, body);
            return rule;
        }
        if (const JsonValue * c = schema.get("const")) return define(name == "root" ? "root" : fresh(name), constant(*c));
        if (const JsonValue * e = schema.get("enum")) {
            if (e->kind != JsonValue::ARRAY || e->items.empty()) throw std::runtime_error("enum must be a list with entries");
            std::string body;
            for (size_t i = 0; i < e->items.size(); ++i) {
                std::string t;
                json_text(e->items[i], t);
                body += (i ? " | " : "") + literal(t);
            }
            return define(name == "root" ? "root" : fresh(name), "( " + body + " ) " + space());
        }
        for (const char * key : {"anyOf", "oneOf"}) {
            if (const JsonValue * alts = schema.get(key)) {
                if (alts->kind != JsonValue::ARRAY || alts->items.empty()) throw std::runtime_error(std::string(key) + " must be a list with entries");
                const std::string rule = name == "root" ? "root" : fresh(name);
                std::string body;
                for (size_t i = 0; i < alts->items.size(); ++i) body += (i ? " | " : "") + visit(alts->items[i], rule + "-" + std::to_string(i));
                return define(rule, body);
            }
        }
        const JsonValue * type = schema.get("type");
        if (type && type->kind == JsonValue::ARRAY) {
            const std::string rule = name == "root" ? "root" : fresh(name);
            std::string body;
            for (size_t i = 0; i < type->items.size(); ++i) {
                JsonValue one = schema;
                for (auto & m : one.members) if (m.first == "type") m.second = type->items[i];
                body += (i ? " | " : "") + visit(one, rule + "-" + type->items[i].text);
            }
            if (body.empty()) throw std::runtime_error("type must name at least one type");
            return define(rule, body);
        }
        std::string t = type && type->kind == JsonValue::STRING ? type->text : "";
        if (t.empty()) {
            if (schema.get("properties") || schema.get("additionalProperties") || schema.get("required")) t = "object";
            else if (schema.get("items") || schema.get("prefixItems")) t = "array";
            else if (schema.get("minLength") || schema.get("maxLength")) t = "string";
            else return any_value();
        }
        if (t == "object") return object(schema, name);
        if (t == "array") return array(schema, name);
        if (t == "string") {
            const JsonValue * lo = schema.get("minLength"), * hi = schema.get("maxLength");
            if (!lo && !hi) return str();
            const long m = lo ? (long)lo->num : 0, n = hi ? (long)hi->num : -1;
            if (m < 0 || (n >= 0 && n < m) || m > 10000 || n > 10000) throw std::runtime_error("minLength / maxLength are out of range");
            chr();
            const std::string rep = n < 0 ? "{" + std::to_string(m) + ",}" : "{" + std::to_string(m) + "," + std::to_string(n) + "}";
            return define(name == "root" ? "root" : fresh(name), "\"\\\"\" char" + rep + " \"\\\"\" " + space());
        }
        if (t == "integer") return integer();
        if (t == "number") return number();
        if (t == "boolean") return boolean();
        if (t == "null") return null();
        throw std::runtime_error("unknown JSON schema type '" + t + "'");
    }

    std::string object(const JsonValue & schema, const std::string & name) {
        const JsonValue * props = schema.get("properties");
        const JsonValue * extra = schema.get("additionalProperties");
        const bool extra_any = extra && ((extra->kind == JsonValue::BOOL && extra->b) || extra->kind == JsonValue::OBJECT);
        if ((!props || props->members.empty()) && (!extra || extra_any) && !schema.get("required")) {
            if (!extra || extra->kind == JsonValue::BOOL) return any_object();
        }
        std::set<std::string> required;
        if (const JsonValue * r = schema.get("required")) {
            if (r->kind != JsonValue::ARRAY) throw std::runtime_error("required must be a list");
            for (const auto & k : r->items) required.insert(k.text);
        }
        const std::string rule = name == "root" ? "root" : fresh(name);
        space();
        // one rule per member: "key" : value
        std::vector<std::string> kv;
        std::vector<bool> must;
        if (props) {
            if (props->kind != JsonValue::OBJECT) throw std::runtime_error("properties must be an object");
            for (const auto & m : props->members) {
                JsonValue key;
                key.kind = JsonValue::STRING;
                key.text = m.first;
                std::string key_text;
                json_text(key, key_text);
                const std::string member = fresh(rule + "-" + m.first);
                const std::string value = visit(m.second, member + "-value");
                define(member, literal(key_text) + " space \":\" space " + value);
                kv.push_back(member);
                must.push_back(required.count(m.first) > 0);
                required.erase(m.first);
            }
        }
        if (!required.empty()) throw std::runtime_error("required names '" + *required.begin() + "', which properties does not declare");
        if (extra_any) {
            str();
            const std::string value = extra->kind == JsonValue::OBJECT ? visit(*extra, rule + "-additional-value") : any_value();
            const std::string member = fresh(rule + "-additional");
            std::vector<std::string> declared;
            if (props) for (const auto & m : props->members) {
                JsonValue key;
                key.kind = JsonValue::STRING;
                key.text = m.first;
                std::string t;
                json_text(key, t);
                declared.push_back(t.substr(1, t.size() - 2));
            }
            define(member, (declared.empty() ? std::string("string") : other_key(rule, declared)) + " \":\" space " + value);
            // any number of further members: an optional member that may repeat
            kv.push_back(member);
            must.push_back(false);
        }
        // after[i]: what may follow once a member has been written, choosing from members i.. in order with every
        // required one present: ("," space member)*. from[i]: the same when nothing has been written yet. The
        // additional member, last if there is one, may repeat. One rule each, so the text stays linear in the
        // number of members.
        const size_t k = kv.size();
        std::vector<std::string> after(k + 1), from(k + 1);
        for (size_t i = k; i-- > 0;) {
            const bool repeat = extra_any && i == k - 1;
            const std::string a_rule = fresh(rule + "-after-" + std::to_string(i));
            const std::string seq = "\",\" space " + kv[i] + (repeat ? " " + a_rule : after[i + 1].empty() ? "" : " " + after[i + 1]);
            if (must[i]) define(a_rule, seq);
            else if (repeat || after[i + 1].empty()) define(a_rule, "( " + seq + " )?");
            else define(a_rule, seq + " | " + after[i + 1]);
            after[i] = a_rule;
        }
        for (size_t i = k; i-- > 0;) {
            const bool repeat = extra_any && i == k - 1;
            const std::string f_rule = fresh(rule + "-from-" + std::to_string(i));
            const std::string seq = kv[i] + (repeat ? " " + after[i] : after[i + 1].empty() ? "" : " " + after[i + 1]);
            if (must[i]) define(f_rule, seq);
            else if (from[i + 1].empty()) define(f_rule, "( " + seq + " )?");
            else define(f_rule, seq + " | " + from[i + 1]);
            from[i] = f_rule;
        }
        return define(rule, "\"{\" space " + (k ? from[0] + " " : std::string()) + "\"}\" space");
    }

    std::string array(const JsonValue & schema, const std::string & name) {
        const std::string rule = name == "root" ? "root" : fresh(name);
        space();
        if (const JsonValue * tuple = schema.get("prefixItems")) {
            if (tuple->kind != JsonValue::ARRAY) throw std::runtime_error("prefixItems must be a list");
            std::string body = "\"[\" space";
            for (size_t i = 0; i < tuple->items.size(); ++i)
                body += std::string(i ? " \",\" space " : " ") + visit(tuple->items[i], rule + "-" + std::to_string(i));
            return define(rule, body + " \"]\" space");
        }
        const JsonValue * items = schema.get("items");
        const std::string item = items ? visit(*items, rule + "-item") : any_value();
        const JsonValue * lo = schema.get("minItems"), * hi = schema.get("maxItems");
        const long m = lo ? (long)lo->num : 0, n = hi ? (long)hi->num : -1;
        if (m < 0 || (n >= 0 && n < m) || m > 10000 || n > 10000) throw std::runtime_error("minItems / maxItems are out of range");
        std::string body = "\"[\" space ";
        if (n == 0) return define(rule, body + "\"]\" space");
        const std::string more = "( \",\" space " + item + " )";
        const std::string rest = n < 0 ? more + "{" + std::to_string(m > 0 ? m - 1 : 0) + ",}"
                                       : more + "{" + std::to_string(m > 0 ? m - 1 : 0) + "," + std::to_string(n - 1) + "}";
        if (m > 0) body += item + " " + rest + " ";
        else body += "( " + item + " " + rest + " )? ";
        return define(rule, body + "\"]\" space");
    }
};

}  // namespace retro
