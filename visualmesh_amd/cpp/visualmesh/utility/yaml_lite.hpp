/*
 * A reader for the subset of YAML that exported Visual Mesh models and dataset lens files use
 * (reference example/load_model.hpp:34-52 and example/dataset.hpp:70-93 read the same files through yaml-cpp;
 * schema written by training/export.py:91-106): block mappings, block sequences (also nested on one line,
 * "- - key: value"), flow sequences and flow mappings (possibly spanning lines), plain and quoted scalars, comments.
 * Anchors, tags, multi-document streams and block scalars are not supported and raise std::runtime_error.
 */
#ifndef VISUALMESH_UTILITY_YAML_LITE_HPP
#define VISUALMESH_UTILITY_YAML_LITE_HPP

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

namespace visualmesh {
namespace yaml {

    class Node {
    public:
        enum Kind { Null, Scalar, Sequence, Mapping };
        Kind kind = Null;
        std::string scalar;
        std::vector<Node> sequence;
        std::vector<std::pair<std::string, Node>> mapping;

        bool defined() const {
            return kind != Null;
        }
        size_t size() const {
            return kind == Sequence ? sequence.size() : kind == Mapping ? mapping.size() : 0;
        }
        const Node& operator[](size_t i) const {
            if (kind != Sequence || i >= sequence.size()) throw std::runtime_error("yaml: sequence index out of range");
            return sequence[i];
        }
        const Node& operator[](const std::string& key) const {
            if (kind != Mapping) throw std::runtime_error("yaml: '" + key + "' looked up in something that is not a mapping");
            for (const auto& kv : mapping)
                if (kv.first == key) return kv.second;
            throw std::runtime_error("yaml: key '" + key + "' not found");
        }
        bool has(const std::string& key) const {
            if (kind != Mapping) return false;
            for (const auto& kv : mapping)
                if (kv.first == key) return true;
            return false;
        }
        std::vector<Node>::const_iterator begin() const {
            return sequence.begin();
        }
        std::vector<Node>::const_iterator end() const {
            return sequence.end();
        }

        const std::string& as_string() const {
            if (kind != Scalar) throw std::runtime_error("yaml: scalar expected");
            return scalar;
        }
        double as_double() const {
            const std::string& s = as_string();
            if (s == ".inf" || s == "+.inf") return HUGE_VAL;
            if (s == "-.inf") return -HUGE_VAL;
            char* end = nullptr;
            const double v = std::strtod(s.c_str(), &end);
            if (end == s.c_str() || *end != '\0') throw std::runtime_error("yaml: '" + s + "' is not a number");
            return v;
        }
        template <typename T>
        std::vector<T> as_vector() const {
            if (kind != Sequence) throw std::runtime_error("yaml: sequence expected");
            std::vector<T> out;
            out.reserve(sequence.size());
            for (const Node& n : sequence) out.push_back(static_cast<T>(n.as_double()));
            return out;
        }
    };

    namespace detail {

        struct Line {
            int indent;
            std::string text;
            int number;
        };

        inline std::string trim(const std::string& s) {
            size_t a = s.find_first_not_of(" \t\r");
            if (a == std::string::npos) return "";
            size_t b = s.find_last_not_of(" \t\r");
            return s.substr(a, b - a + 1);
        }

        /* text up to a comment that starts outside quotes */
        inline std::string strip_comment(const std::string& s) {
            char quote = 0;
            for (size_t i = 0; i < s.size(); ++i) {
                const char c = s[i];
                if (quote) {
                    if (c == quote) quote = 0;
                }
                else if (c == '"' || c == '\'') {
                    quote = c;
                }
                else if (c == '#' && (i == 0 || s[i - 1] == ' ' || s[i - 1] == '\t')) {
                    return s.substr(0, i);
                }
            }
            return s;
        }

        inline std::string unquote(const std::string& s) {
            if (s.size() >= 2 && ((s.front() == '"' && s.back() == '"') || (s.front() == '\'' && s.back() == '\''))) return s.substr(1, s.size() - 2);
            return s;
        }

        inline Node scalar_node(const std::string& raw) {
            Node n;
            const std::string t = trim(raw);
            if (t.empty() || t == "~" || t == "null") return n;
            n.kind = Node::Scalar;
            n.scalar = unquote(t);
            return n;
        }

        /* brackets and braces still open at the end of s (quotes respected) */
        inline int open_brackets(const std::string& s) {
            int depth = 0;
            char quote = 0;
            for (char c : s) {
                if (quote) {
                    if (c == quote) quote = 0;
                }
                else if (c == '"' || c == '\'') quote = c;
                else if (c == '[' || c == '{') ++depth;
                else if (c == ']' || c == '}') --depth;
            }
            return depth;
        }

        /* position of the ':' that ends a mapping key in a block line, or npos */
        inline size_t key_colon(const std::string& s) {
            if (s.empty() || s[0] == '[' || s[0] == '{') return std::string::npos;
            char quote = 0;
            for (size_t i = 0; i < s.size(); ++i) {
                const char c = s[i];
                if (quote) {
                    if (c == quote) quote = 0;
                }
                else if (c == '"' || c == '\'') quote = c;
                else if (c == '[' || c == '{') return std::string::npos;
                else if (c == ':' && (i + 1 == s.size() || s[i + 1] == ' ' || s[i + 1] == '\t')) return i;
            }
            return std::string::npos;
        }

        class FlowParser {
        public:
            explicit FlowParser(const std::string& s) : s(s) {}
            Node parse() {
                Node n = value();
                skip();
                if (i != s.size()) throw std::runtime_error("yaml: unexpected text after flow value: " + s.substr(i));
                return n;
            }

        private:
            const std::string& s;
            size_t i = 0;
            void skip() {
                while (i < s.size() && (s[i] == ' ' || s[i] == '\t' || s[i] == '\n' || s[i] == '\r')) ++i;
            }
            std::string token(const char* stops) {
                skip();
                const size_t start = i;
                if (i < s.size() && (s[i] == '"' || s[i] == '\'')) {
                    const char quote = s[i++];
                    while (i < s.size() && s[i] != quote) ++i;
                    if (i == s.size()) throw std::runtime_error("yaml: unterminated quote");
                    ++i;
                    return s.substr(start, i - start);
                }
                while (i < s.size() && !std::strchr(stops, s[i])) ++i;
                return trim(s.substr(start, i - start));
            }
            Node value() {
                skip();
                if (i >= s.size()) return Node();
                if (s[i] == '[') {
                    ++i;
                    Node n;
                    n.kind = Node::Sequence;
                    skip();
                    if (i < s.size() && s[i] == ']') {
                        ++i;
                        return n;
                    }
                    while (true) {
                        n.sequence.push_back(value());
                        skip();
                        if (i >= s.size()) throw std::runtime_error("yaml: unterminated flow sequence");
                        if (s[i] == ',') {
                            ++i;
                            continue;
                        }
                        if (s[i] == ']') {
                            ++i;
                            return n;
                        }
                        throw std::runtime_error("yaml: ',' or ']' expected in flow sequence");
                    }
                }
                if (s[i] == '{') {
                    ++i;
                    Node n;
                    n.kind = Node::Mapping;
                    skip();
                    if (i < s.size() && s[i] == '}') {
                        ++i;
                        return n;
                    }
                    while (true) {
                        const std::string key = unquote(token(":,}"));
                        skip();
                        if (i >= s.size() || s[i] != ':') throw std::runtime_error("yaml: ':' expected in flow mapping");
                        ++i;
                        n.mapping.emplace_back(key, value());
                        skip();
                        if (i >= s.size()) throw std::runtime_error("yaml: unterminated flow mapping");
                        if (s[i] == ',') {
                            ++i;
                            continue;
                        }
                        if (s[i] == '}') {
                            ++i;
                            return n;
                        }
                        throw std::runtime_error("yaml: ',' or '}' expected in flow mapping");
                    }
                }
                return scalar_node(token(",]}"));
            }
        };

        class BlockParser {
        public:
            explicit BlockParser(std::vector<Line> lines) : lines(std::move(lines)) {}
            Node parse() {
                if (lines.empty()) return Node();
                Node n = block(lines[0].indent);
                if (pos != lines.size()) throw std::runtime_error("yaml: line " + std::to_string(lines[pos].number) + ": unexpected indentation");
                return n;
            }

        private:
            std::vector<Line> lines;
            size_t pos = 0;

            /* an inline value, possibly a flow collection that continues on the following lines */
            Node inline_value(std::string text) {
                if (!text.empty() && (text[0] == '[' || text[0] == '{')) {
                    while (open_brackets(text) > 0) {
                        if (pos >= lines.size()) throw std::runtime_error("yaml: unterminated flow collection");
                        text += " " + lines[pos++].text;
                    }
                    return FlowParser(text).parse();
                }
                if (!text.empty() && (text[0] == '&' || text[0] == '*' || text[0] == '!' || text[0] == '|' || text[0] == '>'))
                    throw std::runtime_error("yaml: anchors, tags and block scalars are not supported");
                return scalar_node(text);
            }

            Node block(int indent) {
                const Line& first = lines[pos];
                if (first.text == "-" || first.text.compare(0, 2, "- ") == 0) return sequence(indent);
                if (key_colon(first.text) != std::string::npos) return mapping(indent);
                std::string text = first.text;
                ++pos;
                return inline_value(text);
            }

            Node sequence(int indent) {
                Node n;
                n.kind = Node::Sequence;
                while (pos < lines.size() && lines[pos].indent == indent && (lines[pos].text == "-" || lines[pos].text.compare(0, 2, "- ") == 0)) {
                    const std::string rest = lines[pos].text.size() > 1 ? lines[pos].text.substr(2) : "";
                    const size_t lead = rest.find_first_not_of(' ');
                    if (lead == std::string::npos) {
                        ++pos;
                        if (pos < lines.size() && lines[pos].indent > indent) n.sequence.push_back(block(lines[pos].indent));
                        else n.sequence.push_back(Node());
                    }
                    else {
                        /* the item starts on this line: treat the remainder as a line of its own, indented past the dash */
                        lines[pos].indent = indent + 2 + int(lead);
                        lines[pos].text = rest.substr(lead);
                        n.sequence.push_back(block(lines[pos].indent));
                    }
                }
                return n;
            }

            Node mapping(int indent) {
                Node n;
                n.kind = Node::Mapping;
                while (pos < lines.size() && lines[pos].indent == indent) {
                    const std::string text = lines[pos].text;
                    const size_t colon = key_colon(text);
                    if (colon == std::string::npos) throw std::runtime_error("yaml: line " + std::to_string(lines[pos].number) + ": mapping key expected");
                    const std::string key = unquote(trim(text.substr(0, colon)));
                    const std::string rest = trim(text.substr(colon + 1));
                    ++pos;
                    if (rest.empty()) {
                        /* the value is the following block; a sequence may sit at the key's own indentation */
                        if (pos < lines.size()
                            && (lines[pos].indent > indent
                                || (lines[pos].indent == indent && (lines[pos].text == "-" || lines[pos].text.compare(0, 2, "- ") == 0))))
                            n.mapping.emplace_back(key, block(lines[pos].indent));
                        else n.mapping.emplace_back(key, Node());
                    }
                    else {
                        n.mapping.emplace_back(key, inline_value(rest));
                    }
                }
                return n;
            }
        };

    }  // namespace detail

    inline Node parse(const std::string& document) {
        std::vector<detail::Line> lines;
        std::istringstream in(document);
        std::string raw;
        int number = 0;
        while (std::getline(in, raw)) {
            ++number;
            if (raw.compare(0, 3, "---") == 0 && lines.empty()) continue; /* a single document marker */
            std::string text = detail::strip_comment(raw);
            const size_t lead = text.find_first_not_of(' ');
            if (lead == std::string::npos || detail::trim(text).empty()) continue;
            if (text.find('\t') != std::string::npos && text.find('\t') < lead + 1) throw std::runtime_error("yaml: tabs cannot indent");
            lines.push_back({int(lead), detail::trim(text), number});
        }
        return detail::BlockParser(std::move(lines)).parse();
    }

    inline Node load_file(const std::string& path) {
        std::ifstream in(path);
        if (!in) throw std::runtime_error("yaml: cannot open " + path);
        std::ostringstream text;
        text << in.rdbuf();
        return parse(text.str());
    }

}  // namespace yaml
}  // namespace visualmesh

#endif  // VISUALMESH_UTILITY_YAML_LITE_HPP
