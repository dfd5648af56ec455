#include "json.h"

#include <cstdlib>
#include <sstream>

#include "../log.h"

namespace chainer_compiler {

class JsonParser {
public:
    explicit JsonParser(const std::string& text) : s_(text) {
    }

    Json ParseDocument() {
        Json v = ParseValue();
        SkipSpace();
        CHECK_EQ(pos_, s_.size()) << "trailing characters in JSON at offset " << pos_;
        return v;
    }

private:
    void SkipSpace() {
        for (;;) {
            while (pos_ < s_.size() && (s_[pos_] == ' ' || s_[pos_] == '\t' || s_[pos_] == '\n' || s_[pos_] == '\r')) ++pos_;
            if (pos_ + 1 < s_.size() && s_[pos_] == '/' && s_[pos_ + 1] == '/') {
                while (pos_ < s_.size() && s_[pos_] != '\n') ++pos_;
                continue;
            }
            return;
        }
    }

    char Peek() {
        SkipSpace();
        CHECK_LT(pos_, s_.size()) << "unexpected end of JSON";
        return s_[pos_];
    }

    void Expect(char c) {
        CHECK_EQ(Peek(), c) << "JSON syntax error at offset " << pos_;
        ++pos_;
    }

    bool Consume(const char* word) {
        const size_t n = std::char_traits<char>::length(word);
        if (s_.compare(pos_, n, word) != 0) return false;
        pos_ += n;
        return true;
    }

    std::string ParseString() {
        Expect('"');
        std::string out;
        while (true) {
            CHECK_LT(pos_, s_.size()) << "unterminated JSON string";
            char c = s_[pos_++];
            if (c == '"') break;
            if (c != '\\') {
                out.push_back(c);
                continue;
            }
            CHECK_LT(pos_, s_.size()) << "unterminated JSON escape";
            c = s_[pos_++];
            switch (c) {
                case 'n': out.push_back('\n'); break;
                case 't': out.push_back('\t'); break;
                case 'r': out.push_back('\r'); break;
                case 'b': out.push_back('\b'); break;
                case 'f': out.push_back('\f'); break;
                case 'u': {
                    CHECK_LE(pos_ + 4, s_.size()) << "short \\u escape";
                    const unsigned cp = static_cast<unsigned>(std::strtoul(s_.substr(pos_, 4).c_str(), nullptr, 16));
                    pos_ += 4;
                    if (cp < 0x80) {
                        out.push_back(static_cast<char>(cp));
                    } else if (cp < 0x800) {
                        out.push_back(static_cast<char>(0xC0 | (cp >> 6)));
                        out.push_back(static_cast<char>(0x80 | (cp & 0x3F)));
                    } else {
                        out.push_back(static_cast<char>(0xE0 | (cp >> 12)));
                        out.push_back(static_cast<char>(0x80 | ((cp >> 6) & 0x3F)));
                        out.push_back(static_cast<char>(0x80 | (cp & 0x3F)));
                    }
                } break;
                default: out.push_back(c);  // \" \\ \/
            }
        }
        return out;
    }

    Json ParseValue() {
        Json v;
        const char c = Peek();
        if (c == '{') {
            ++pos_;
            v.kind_ = Json::Kind::kObject;
            if (Peek() == '}') {
                ++pos_;
                return v;
            }
            while (true) {
                SkipSpace();
                std::string key = ParseString();
                Expect(':');
                Json member = ParseValue();
                CHECK(v.object_.emplace(key, std::move(member)).second) << "Duplicate key: " << key;
                if (Peek() == ',') {
                    ++pos_;
                    continue;
                }
                Expect('}');
                break;
            }
        } else if (c == '[') {
            ++pos_;
            v.kind_ = Json::Kind::kArray;
            if (Peek() == ']') {
                ++pos_;
                return v;
            }
            while (true) {
                v.array_.push_back(ParseValue());
                if (Peek() == ',') {
                    ++pos_;
                    continue;
                }
                Expect(']');
                break;
            }
        } else if (c == '"') {
            v.kind_ = Json::Kind::kString;
            v.string_ = ParseString();
        } else if (Consume("true")) {
            v.kind_ = Json::Kind::kBool;
            v.bool_ = true;
        } else if (Consume("false")) {
            v.kind_ = Json::Kind::kBool;
        } else if (Consume("null")) {
            // stays null
        } else {
            const char* begin = s_.c_str() + pos_;
            char* end = nullptr;
            v.number_ = std::strtod(begin, &end);
            CHECK(end != begin) << "JSON syntax error at offset " << pos_;
            v.kind_ = Json::Kind::kNumber;
            pos_ += static_cast<size_t>(end - begin);
        }
        return v;
    }

    const std::string& s_;
    size_t pos_ = 0;
};

Json Json::Parse(const std::string& text) {
    return JsonParser(text).ParseDocument();
}

const Json* Json::find(const std::string& key) const {
    if (!is_object()) return nullptr;
    auto it = object_.find(key);
    return it == object_.end() ? nullptr : &it->second;
}

void Json::merge_patch(const Json& patch) {
    if (!patch.is_object()) {
        *this = patch;
        return;
    }
    if (!is_object()) {
        *this = Json();
        kind_ = Kind::kObject;
    }
    for (const auto& el : patch.object_) {
        if (el.second.is_null()) {
            object_.erase(el.first);
        } else {
            object_[el.first].merge_patch(el.second);
        }
    }
}

std::string Json::dump() const {
    std::ostringstream oss;
    switch (kind_) {
        case Kind::kNull: oss << "null"; break;
        case Kind::kBool: oss << (bool_ ? "true" : "false"); break;
        case Kind::kNumber: oss << number_; break;
        case Kind::kString: oss << '"' << string_ << '"'; break;
        case Kind::kArray: {
            oss << '[';
            for (size_t i = 0; i < array_.size(); ++i) oss << (i ? "," : "") << array_[i].dump();
            oss << ']';
        } break;
        case Kind::kObject: {
            oss << '{';
            bool first = true;
            for (const auto& el : object_) {
                oss << (first ? "" : ",") << '"' << el.first << "\":" << el.second.dump();
                first = false;
            }
            oss << '}';
        } break;
    }
    return oss.str();
}

}  // namespace chainer_compiler
