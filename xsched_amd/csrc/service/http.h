// A small HTTP/1.1 responder and the flat JSON it needs: enough for the scheduler daemon's
// control plane (a handful of GET / POST routes with query parameters or a one-level JSON
// body, answered with a JSON object). One thread, one connection at a time, every response
// closes its connection. The reference's daemon uses the cpp-httplib and jsoncpp libraries for
// this (service/server/src/server.cpp:28-39,270-543), which are not part of its source tree.
#pragma once

#include <atomic>
#include <cstdint>
#include <functional>
#include <map>
#include <string>
#include <thread>

namespace xsched::service
{

struct HttpRequest
{
    std::string method;                          // "GET", "POST"
    std::string path;                            // without the query string, percent-decoded
    std::map<std::string, std::string> query;    // ?a=b&c=d, percent-decoded
    std::string body;
};

struct HttpResponse
{
    int status = 200;
    std::string body;                            // JSON text, may be empty
};

using HttpHandler = std::function<void(const HttpRequest &, HttpResponse &)>;

class HttpServer
{
public:
    HttpServer() = default;
    ~HttpServer() { Stop(); }

    /// Binds and starts the serving thread. False (with a warning) when the port cannot be bound.
    bool Start(const std::string &address, int port, HttpHandler handler);
    void Stop();
    int Port() const { return port_; }

private:
    void Serve();
    void ServeOne(int fd);

    int listen_fd_ = -1;
    int port_ = 0;
    std::atomic<bool> stop_ { false };
    HttpHandler handler_;
    std::thread thread_;
};

// ---- flat JSON ----------------------------------------------------------------------------

/// Builds one JSON value as text. Numbers are written in full (64-bit handles do not fit a
/// double).
class JsonWriter
{
public:
    static std::string Quote(const std::string &s);

    JsonWriter &BeginObject() { Sep(); out_ += '{'; first_ = true; return *this; }
    JsonWriter &EndObject()   { out_ += '}'; first_ = false; return *this; }
    JsonWriter &BeginArray()  { Sep(); out_ += '['; first_ = true; return *this; }
    JsonWriter &EndArray()    { out_ += ']'; first_ = false; return *this; }
    JsonWriter &Key(const std::string &k) { Sep(); out_ += Quote(k); out_ += ':'; first_ = true; return *this; }
    JsonWriter &UInt(uint64_t v)  { Sep(); out_ += std::to_string(v); return *this; }
    JsonWriter &Int(int64_t v)    { Sep(); out_ += std::to_string(v); return *this; }
    JsonWriter &Bool(bool v)      { Sep(); out_ += v ? "true" : "false"; return *this; }
    JsonWriter &String(const std::string &v) { Sep(); out_ += Quote(v); return *this; }
    const std::string &Text() const { return out_; }

private:
    void Sep() { if (!first_) out_ += ','; first_ = false; }
    std::string out_;
    bool first_ = true;
};

/// One level of {"key": value, ...}: integers keep all their digits, strings are unescaped,
/// true / false / null are kept as words. False when the text is not such an object.
bool ParseFlatJsonObject(const std::string &text, std::map<std::string, std::string> *out);

/// Whole-string conversions; false on anything else than a number in range.
bool ParseUInt64(const std::string &s, int base, uint64_t *out);
bool ParseInt64(const std::string &s, int64_t *out);

} // namespace xsched::service
