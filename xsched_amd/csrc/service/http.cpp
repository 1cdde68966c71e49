// See http.h.
#include <algorithm>
#include <arpa/inet.h>
#include <cerrno>
#include <chrono>
#include <cstring>
#include <netinet/in.h>
#include <poll.h>
#include <sys/socket.h>
#include <unistd.h>

#include "http.h"
#include "xsched/utils/log.h"

namespace xsched::service
{

namespace
{

constexpr size_t kMaxRequestBytes = 1 << 16;
constexpr int kRequestDeadlineSeconds = 3;   // for a whole request, headers and body

int HexDigit(char c)
{
    if (c >= '0' && c <= '9') return c - '0';
    if (c >= 'a' && c <= 'f') return c - 'a' + 10;
    if (c >= 'A' && c <= 'F') return c - 'A' + 10;
    return -1;
}

std::string PercentDecode(const std::string &s, bool plus_is_space)
{
    std::string out;
    for (size_t i = 0; i < s.size(); ++i) {
        if (s[i] == '%' && i + 2 < s.size() && HexDigit(s[i + 1]) >= 0 && HexDigit(s[i + 2]) >= 0) {
            out += (char)(HexDigit(s[i + 1]) * 16 + HexDigit(s[i + 2]));
            i += 2;
        } else if (s[i] == '+' && plus_is_space) {
            out += ' ';
        } else {
            out += s[i];
        }
    }
    return out;
}

const char *Reason(int status)
{
    switch (status) {
    case 200: return "OK";
    case 400: return "Bad Request";
    case 404: return "Not Found";
    case 405: return "Method Not Allowed";
    case 408: return "Request Timeout";
    case 413: return "Payload Too Large";
    default:  return "Internal Server Error";
    }
}

bool SendAll(int fd, const std::string &data)
{
    size_t sent = 0;
    while (sent < data.size()) {
        const ssize_t n = send(fd, data.data() + sent, data.size() - sent, MSG_NOSIGNAL);
        if (n < 0) { if (errno == EINTR) continue; return false; }
        sent += (size_t)n;
    }
    return true;
}

std::string Lower(std::string s)
{
    for (char &c : s) if (c >= 'A' && c <= 'Z') c = (char)(c - 'A' + 'a');
    return s;
}

} // namespace

bool HttpServer::Start(const std::string &address, int port, HttpHandler handler)
{
    handler_ = std::move(handler);
    listen_fd_ = socket(AF_INET, SOCK_STREAM | SOCK_CLOEXEC, 0);
    if (listen_fd_ < 0) { XWARN("http: socket() failed: %s", strerror(errno)); return false; }
    int one = 1;
    setsockopt(listen_fd_, SOL_SOCKET, SO_REUSEADDR, &one, sizeof(one));
    sockaddr_in addr {};
    addr.sin_family = AF_INET;
    addr.sin_port = htons((uint16_t)port);
    if (inet_pton(AF_INET, address.c_str(), &addr.sin_addr) != 1) {
        XWARN("http: '%s' is not an IPv4 address", address.c_str());
        close(listen_fd_); listen_fd_ = -1;
        return false;
    }
    if (bind(listen_fd_, (sockaddr *)&addr, sizeof(addr)) != 0 || listen(listen_fd_, 16) != 0) {
        XWARN("http: cannot listen on %s:%d: %s", address.c_str(), port, strerror(errno));
        close(listen_fd_); listen_fd_ = -1;
        return false;
    }
    socklen_t len = sizeof(addr);
    if (getsockname(listen_fd_, (sockaddr *)&addr, &len) == 0) port_ = ntohs(addr.sin_port);
    stop_.store(false);
    thread_ = std::thread([this]() { Serve(); });
    return true;
}

void HttpServer::Stop()
{
    stop_.store(true);
    if (thread_.joinable()) thread_.join();
    if (listen_fd_ >= 0) { close(listen_fd_); listen_fd_ = -1; }
}

void HttpServer::Serve()
{
    while (!stop_.load()) {
        pollfd pfd { listen_fd_, POLLIN, 0 };
        const int rc = poll(&pfd, 1, 100);
        if (rc <= 0 || !(pfd.revents & POLLIN)) continue;
        const int fd = accept4(listen_fd_, nullptr, nullptr, SOCK_CLOEXEC);
        if (fd < 0) continue;
        timeval tv { 2, 0 };   // a client that stops talking does not hold the only serving thread
        setsockopt(fd, SOL_SOCKET, SO_RCVTIMEO, &tv, sizeof(tv));
        setsockopt(fd, SOL_SOCKET, SO_SNDTIMEO, &tv, sizeof(tv));
        ServeOne(fd);
        close(fd);
    }
}

void HttpServer::ServeOne(int fd)
{
    // One thread serves every client, so a request has a deadline as a whole, not only per
    // read: a client that sends a byte every second would otherwise hold the control plane
    // (and Stop()) for as long as it likes. Past the deadline it is answered 408 and dropped.
    const auto deadline = std::chrono::steady_clock::now() + std::chrono::seconds(kRequestDeadlineSeconds);
    bool timed_out = false;
    auto read_more = [&](char *into, size_t cap) -> ssize_t {
        while (true) {
            const auto left = std::chrono::duration_cast<std::chrono::milliseconds>(deadline - std::chrono::steady_clock::now()).count();
            if (left <= 0 || stop_.load()) { timed_out = true; return -1; }
            pollfd pfd { fd, POLLIN, 0 };
            const int rc = poll(&pfd, 1, (int)std::min<int64_t>(left, 100));
            if (rc < 0 && errno != EINTR) return -1;
            if (rc > 0) return recv(fd, into, cap, 0);
        }
    };
    std::string raw;
    size_t header_end = std::string::npos;
    char buf[4096];
    HttpResponse res;
    HttpRequest req;
    auto reply = [&]() {
        std::string head = "HTTP/1.1 " + std::to_string(res.status) + " " + Reason(res.status) + "\r\n";
        if (!res.body.empty()) head += "Content-Type: application/json\r\n";
        head += "Content-Length: " + std::to_string(res.body.size()) + "\r\nConnection: close\r\n\r\n";
        SendAll(fd, head + res.body);
    };
    while (header_end == std::string::npos && raw.size() < kMaxRequestBytes) {
        const ssize_t n = read_more(buf, sizeof(buf));
        if (n <= 0) { if (timed_out) { res.status = 408; reply(); } return; }
        raw.append(buf, (size_t)n);
        header_end = raw.find("\r\n\r\n");
    }
    if (header_end == std::string::npos) { res.status = 413; reply(); return; }

    // request line
    const size_t line_end = raw.find("\r\n");
    const std::string line = raw.substr(0, line_end);
    const size_t sp1 = line.find(' '), sp2 = line.rfind(' ');
    if (sp1 == std::string::npos || sp2 == sp1) { res.status = 400; reply(); return; }
    req.method = line.substr(0, sp1);
    std::string target = line.substr(sp1 + 1, sp2 - sp1 - 1);
    const size_t q = target.find('?');
    req.path = PercentDecode(target.substr(0, q), false);
    if (q != std::string::npos) {
        std::string qs = target.substr(q + 1);
        size_t pos = 0;
        while (pos <= qs.size()) {
            size_t amp = qs.find('&', pos);
            if (amp == std::string::npos) amp = qs.size();
            const std::string pair = qs.substr(pos, amp - pos);
            if (!pair.empty()) {
                const size_t eq = pair.find('=');
                const std::string k = PercentDecode(pair.substr(0, eq), true);
                req.query[k] = eq == std::string::npos ? "" : PercentDecode(pair.substr(eq + 1), true);
            }
            pos = amp + 1;
        }
    }
    // headers: only the body's length matters
    size_t content_length = 0;
    size_t pos = line_end + 2;
    while (pos < header_end) {
        size_t eol = raw.find("\r\n", pos);
        if (eol == std::string::npos || eol > header_end) eol = header_end;
        const std::string h = raw.substr(pos, eol - pos);
        const size_t colon = h.find(':');
        if (colon != std::string::npos && Lower(h.substr(0, colon)) == "content-length") {
            uint64_t v = 0;
            std::string num = h.substr(colon + 1);
            num.erase(0, num.find_first_not_of(" \t"));
            num.erase(num.find_last_not_of(" \t") + 1);
            if (!ParseUInt64(num, 10, &v) || v > kMaxRequestBytes) { res.status = 413; reply(); return; }
            content_length = (size_t)v;
        }
        pos = eol + 2;
    }
    req.body = raw.substr(header_end + 4);
    while (req.body.size() < content_length) {
        const ssize_t n = read_more(buf, sizeof(buf));
        if (n <= 0) { if (timed_out) { res.status = 408; reply(); } return; }
        req.body.append(buf, (size_t)n);
    }
    req.body.resize(content_length);

    handler_(req, res);
    reply();
}

// ---- flat JSON ----------------------------------------------------------------------------

std::string JsonWriter::Quote(const std::string &s)
{
    std::string out = "\"";
    for (unsigned char c : s) {
        switch (c) {
        case '"':  out += "\\\""; break;
        case '\\': out += "\\\\"; break;
        case '\n': out += "\\n"; break;
        case '\r': out += "\\r"; break;
        case '\t': out += "\\t"; break;
        default:
            if (c < 0x20) { char u[8]; snprintf(u, sizeof(u), "\\u%04x", c); out += u; }
            else out += (char)c;
        }
    }
    return out + "\"";
}

bool ParseUInt64(const std::string &s, int base, uint64_t *out)
{
    if (s.empty() || s[0] == '-' || s[0] == '+' || s[0] == ' ') return false;
    errno = 0;
    char *end = nullptr;
    const unsigned long long v = strtoull(s.c_str(), &end, base);
    if (errno != 0 || end != s.c_str() + s.size()) return false;
    *out = v;
    return true;
}

bool ParseInt64(const std::string &s, int64_t *out)
{
    if (s.empty() || s[0] == ' ' || s[0] == '+') return false;
    errno = 0;
    char *end = nullptr;
    const long long v = strtoll(s.c_str(), &end, 10);
    if (errno != 0 || end != s.c_str() + s.size()) return false;
    *out = v;
    return true;
}

bool ParseFlatJsonObject(const std::string &text, std::map<std::string, std::string> *out)
{
    size_t i = 0;
    auto skip = [&]() { while (i < text.size() && (text[i] == ' ' || text[i] == '\t' || text[i] == '\n' || text[i] == '\r')) ++i; };
    auto string = [&](std::string *s) {
        if (i >= text.size() || text[i] != '"') return false;
        ++i;
        while (i < text.size() && text[i] != '"') {
            if (text[i] == '\\') {
                if (++i >= text.size()) return false;
                switch (text[i]) {
                case 'n': *s += '\n'; break;
                case 't': *s += '\t'; break;
                case 'r': *s += '\r'; break;
                case 'b': *s += '\b'; break;
                case 'f': *s += '\f'; break;
                case 'u':
                {
                    if (i + 4 >= text.size()) return false;
                    unsigned code = 0;
                    for (int k = 1; k <= 4; ++k) { const int d = HexDigit(text[i + k]); if (d < 0) return false; code = code * 16 + (unsigned)d; }
                    *s += code < 0x80 ? (char)code : '?';
                    i += 4;
                    break;
                }
                default: *s += text[i];
                }
            } else {
                *s += text[i];
            }
            ++i;
        }
        if (i >= text.size()) return false;
        ++i;
        return true;
    };
    skip();
    if (i >= text.size() || text[i] != '{') return false;
    ++i;
    skip();
    if (i < text.size() && text[i] == '}') { ++i; skip(); return i == text.size(); }
    while (true) {
        skip();
        std::string key, value;
        if (!string(&key)) return false;
        skip();
        if (i >= text.size() || text[i] != ':') return false;
        ++i;
        skip();
        if (i < text.size() && text[i] == '"') {
            if (!string(&value)) return false;
        } else {
            const size_t start = i;
            while (i < text.size() && text[i] != ',' && text[i] != '}' && text[i] != ' ' && text[i] != '\n' &&
                   text[i] != '\r' && text[i] != '\t') ++i;
            value = text.substr(start, i - start);
            if (value.empty() || value[0] == '{' || value[0] == '[') return false; // one level only
        }
        (*out)[key] = value;
        skip();
        if (i < text.size() && text[i] == ',') { ++i; continue; }
        if (i < text.size() && text[i] == '}') { ++i; break; }
        return false;
    }
    skip();
    return i == text.size();
}

} // namespace xsched::service
