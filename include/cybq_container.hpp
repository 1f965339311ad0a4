// cybq_container.hpp - reader of the .cyb / .model container for quantised
// weights (header only, POSIX mmap).
//
// Container rules: /root/reference/reference/format.md:14-20 (TOML frontmatter
// until the first `~~~`; `~~~name` + LF separates every file inside; binary
// files have `size`), :33-35 (LF only), :78-84 (text before binary, text runs to
// the next `~~~`), :110-117 (order = order of [[files]]).  The file is mapped,
// not read (/root/reference/shell/src/lib.rs:31-33).
//
// The record format of the tensor index is this build's (the reference's is not
// in its tree): a text part `tensors` holding [[tensor]] tables
//   name, kind = "q4"|"q8", layout = "block_aos"|"planar", shape = [N, K],
//   offset, nbytes, and scales_offset / scales_nbytes for planar
// that point into one binary part `weights`.
//
// The TOML reader below understands the subset those two texts use: [table],
// [[array of tables]], key = "string" | integer | [integers] | ["strings"].
#pragma once

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <utility>
#include <vector>

#include "cybq.hpp"

namespace cybq {

struct TomlTable {
    std::string name;                                   // "cyb", "files", "tensor", ... ("" = root)
    std::map<std::string, std::string> str;             // string values
    std::map<std::string, std::vector<int64_t>> ints;   // integers and integer arrays
};

// Parses the subset described above; returns false and sets `err` on anything else.
inline bool parse_toml_subset(const char* p, size_t n, std::vector<TomlTable>& out, std::string& err)
{
    out.clear();
    out.push_back(TomlTable{});
    size_t i = 0;
    int line_no = 0;
    auto trim = [](std::string s) {
        size_t a = s.find_first_not_of(" \t\r"), b = s.find_last_not_of(" \t\r");
        return a == std::string::npos ? std::string() : s.substr(a, b - a + 1);
    };
    while (i < n) {
        size_t e = i;
        while (e < n && p[e] != '\n') e++;
        std::string line = trim(std::string(p + i, e - i));
        i = e + 1;
        line_no++;
        if (line.empty() || line[0] == '#') continue;
        if (line[0] == '[') {
            bool arr = line.size() > 1 && line[1] == '[';
            size_t close = line.find(arr ? "]]" : "]");
            if (close == std::string::npos) { err = "line " + std::to_string(line_no) + ": bad table header"; return false; }
            TomlTable t;
            t.name = trim(line.substr(arr ? 2 : 1, close - (arr ? 2 : 1)));
            out.push_back(t);
            continue;
        }
        size_t eq = line.find('=');
        if (eq == std::string::npos) { err = "line " + std::to_string(line_no) + ": expected key = value"; return false; }
        std::string key = trim(line.substr(0, eq)), val = trim(line.substr(eq + 1));
        if (key.empty() || val.empty()) { err = "line " + std::to_string(line_no) + ": empty key or value"; return false; }
        TomlTable& t = out.back();
        auto parse_string = [&](const std::string& v, size_t& pos, std::string& s) {
            if (v[pos] != '"') return false;
            s.clear();
            for (pos++; pos < v.size(); pos++) {
                if (v[pos] == '\\' && pos + 1 < v.size()) { s.push_back(v[++pos]); continue; }
                if (v[pos] == '"') { pos++; return true; }
                s.push_back(v[pos]);
            }
            return false;
        };
        if (val[0] == '"') {
            size_t pos = 0;
            std::string s;
            if (!parse_string(val, pos, s)) { err = "line " + std::to_string(line_no) + ": bad string"; return false; }
            t.str[key] = s;
        } else if (val[0] == '[') {
            std::vector<int64_t> v;
            size_t pos = 1;
            bool strings = false;
            while (pos < val.size() && val[pos] != ']') {
                while (pos < val.size() && (val[pos] == ' ' || val[pos] == ',')) pos++;
                if (pos >= val.size() || val[pos] == ']') break;
                if (val[pos] == '"') {
                    std::string s;
                    if (!parse_string(val, pos, s)) { err = "line " + std::to_string(line_no) + ": bad string array"; return false; }
                    t.str[key] += (strings ? "," : "") + s;
                    strings = true;
                } else {
                    char* endp = nullptr;
                    long long x = std::strtoll(val.c_str() + pos, &endp, 10);
                    if (endp == val.c_str() + pos) { err = "line " + std::to_string(line_no) + ": bad array element"; return false; }
                    v.push_back(x);
                    pos = (size_t)(endp - val.c_str());
                }
            }
            if (!strings) t.ints[key] = v;
        } else {
            char* endp = nullptr;
            long long x = std::strtoll(val.c_str(), &endp, 10);
            if (endp == val.c_str()) { err = "line " + std::to_string(line_no) + ": unsupported value '" + val + "'"; return false; }
            t.ints[key] = {x};
        }
    }
    return true;
}

struct TensorRecord {
    std::string name;
    cybq_quant quant = CYBQ_Q4;
    cybq_layout layout = CYBQ_LAYOUT_BLOCK_AOS;
    int64_t N = 0, K = 0;
    const uint8_t* q = nullptr;          // into the mapping
    const uint8_t* scales = nullptr;     // planar only
};

class Container {
public:
    Container() = default;
    Container(const Container&) = delete;
    Container& operator=(const Container&) = delete;
    ~Container() { close(); }

    Status open(const std::string& path)
    {
        close();
        fd_ = ::open(path.c_str(), O_RDONLY);
        if (fd_ < 0) return bad("cannot open " + path);
        struct stat st;
        if (fstat(fd_, &st) != 0 || st.st_size <= 0) return bad("empty or unreadable file");
        size_ = (size_t)st.st_size;
        void* m = mmap(nullptr, size_, PROT_READ, MAP_PRIVATE, fd_, 0);
        if (m == MAP_FAILED) { map_ = nullptr; return bad("mmap failed"); }
        map_ = static_cast<const uint8_t*>(m);
        return parse();
    }
    void close()
    {
        if (map_) munmap(const_cast<uint8_t*>(map_), size_);
        if (fd_ >= 0) ::close(fd_);
        map_ = nullptr; fd_ = -1; size_ = 0;
        parts_.clear(); tensors_.clear();
    }
    const std::string& name() const { return name_; }
    const std::vector<TensorRecord>& tensors() const { return tensors_; }
    // (pointer, length) of a part; pointer is null when the part does not exist
    std::pair<const uint8_t*, size_t> part(const std::string& n) const
    {
        auto it = parts_.find(n);
        if (it == parts_.end()) return {nullptr, 0};
        return {map_ + it->second.first, it->second.second};
    }

    // uploads every tensor into the backend under its name (model load)
    Status load_into(Backend& be) const
    {
        for (const auto& t : tensors_) {
            Status s = be.load(t.name, t.quant, t.layout, t.N, t.K, t.q, t.scales);
            if (!s) return s;
        }
        return Status{};
    }

private:
    Status bad(const std::string& why) const { Status s; s.code = CYBQ_ERR_INVALID; s.text = "container: " + why; return s; }

    // first `~~~` at the start of a line at or after `from`; size_ when there is none
    size_t find_delim(size_t from) const
    {
        for (size_t i = from; i + 3 <= size_; i++)
            if (map_[i] == '~' && map_[i + 1] == '~' && map_[i + 2] == '~' && (i == 0 || map_[i - 1] == '\n')) return i;
        return size_;
    }

    Status parse()
    {
        size_t first = find_delim(0);
        if (first == size_) return bad("no ~~~ delimiter");
        std::vector<TomlTable> front;
        std::string err;
        if (!parse_toml_subset(reinterpret_cast<const char*>(map_), first, front, err)) return bad("frontmatter " + err);
        size_t pos = first;
        bool seen_binary = false, any = false;
        size_t files_left = 0;
        for (const auto& t : front) files_left += t.name == "files";
        for (const auto& t : front) {
            if (t.name == "cyb") { auto it = t.str.find("name"); if (it != t.str.end()) name_ = it->second; }
            if (t.name != "files") continue;
            any = true;
            files_left--;
            auto nm = t.str.find("name");
            if (nm == t.str.end()) return bad("a [[files]] entry has no name");
            std::string head = "~~~" + nm->second + "\n";
            if (pos + head.size() > size_ || std::memcmp(map_ + pos, head.data(), head.size()) != 0)
                return bad("expected delimiter ~~~" + nm->second);
            size_t body = pos + head.size();
            auto sz = t.ints.find("size");
            if (sz != t.ints.end() && !sz->second.empty()) {
                seen_binary = true;
                int64_t n = sz->second[0];
                if (n < 0 || body + (size_t)n > size_) return bad("part '" + nm->second + "' runs past the end of the file");
                parts_[nm->second] = {body, (size_t)n};
                pos = body + (size_t)n;
            } else {
                if (seen_binary) {
                    // text goes before binary; a LAST part without a size runs to the end of the file
                    // (/root/reference/reference/format.md:24-31)
                    if (files_left != 0) return bad("text part '" + nm->second + "' after a binary part");
                    parts_[nm->second] = {body, size_ - body};
                    pos = size_;
                    continue;
                }
                size_t end = find_delim(body);
                parts_[nm->second] = {body, end - body};
                pos = end;
            }
        }
        if (!any) return bad("frontmatter lists no [[files]]");
        auto ti = parts_.find("tensors"), wi = parts_.find("weights");
        if (ti == parts_.end() || wi == parts_.end()) return Status{};      // a container without weights is valid
        std::vector<TomlTable> idx;
        if (!parse_toml_subset(reinterpret_cast<const char*>(map_ + ti->second.first), ti->second.second, idx, err))
            return bad("tensor index " + err);
        const uint8_t* wbase = map_ + wi->second.first;
        const size_t wlen = wi->second.second;
        for (const auto& t : idx) {
            if (t.name != "tensor") continue;
            TensorRecord r;
            auto s = [&](const char* k) { auto it = t.str.find(k); return it == t.str.end() ? std::string() : it->second; };
            auto iv = [&](const char* k, size_t j) -> int64_t {
                auto it = t.ints.find(k);
                return (it == t.ints.end() || it->second.size() <= j) ? -1 : it->second[j];
            };
            r.name = s("name");
            std::string kind = s("kind"), layout = s("layout");
            if (r.name.empty() || (kind != "q4" && kind != "q8") || (layout != "planar" && layout != "block_aos"))
                return bad("bad tensor record '" + r.name + "'");
            r.quant = kind == "q4" ? CYBQ_Q4 : CYBQ_Q8;
            r.layout = layout == "planar" ? CYBQ_LAYOUT_PLANAR : CYBQ_LAYOUT_BLOCK_AOS;
            r.N = iv("shape", 0);
            r.K = iv("shape", 1);
            int64_t off = iv("offset", 0), nb = iv("nbytes", 0);
            if (r.N < 1 || r.K < 1 || r.K % CYBQ_GROUP || off < 0 || nb < 0) return bad("tensor '" + r.name + "': bad shape or offset");
            const int64_t groups = r.N * (r.K / CYBQ_GROUP);
            const int64_t want = r.layout == CYBQ_LAYOUT_BLOCK_AOS ? groups * (r.quant == CYBQ_Q4 ? 18 : 34)
                                                                    : r.N * r.K * (int)r.quant / 8;
            if (nb != want || (size_t)(off + nb) > wlen) return bad("tensor '" + r.name + "': payload does not fit");
            r.q = wbase + off;
            if (r.layout == CYBQ_LAYOUT_PLANAR) {
                int64_t so = iv("scales_offset", 0), sn = iv("scales_nbytes", 0);
                if (so < 0 || sn != groups * 2 || (size_t)(so + sn) > wlen) return bad("tensor '" + r.name + "': scale plane does not fit");
                r.scales = wbase + so;
            }
            tensors_.push_back(r);
        }
        return Status{};
    }

    int fd_ = -1;
    const uint8_t* map_ = nullptr;
    size_t size_ = 0;
    std::string name_;
    std::map<std::string, std::pair<size_t, size_t>> parts_;
    std::vector<TensorRecord> tensors_;
};

}  // namespace cybq
