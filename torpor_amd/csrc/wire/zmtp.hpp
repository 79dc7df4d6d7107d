// ZMTP 3.0 (ZeroMQ Message Transport Protocol, rfc.zeromq.org/spec/23) over AF_UNIX stream
// sockets, NULL security mechanism: what libzmq speaks on an `ipc://` endpoint.  The reference
// links libzmq 4.2.5 (common/vendor/zeromq/CMakeLists.txt:20-21) and uses REQ/REP for control
// signals and PUSH/PULL for the data plane (common/include/socket_helper.hpp:10-32,
// include/server/controller.hpp:56,77, include/server/cuda_server.hpp:51-53); libzmq is not part
// of the ROCm image, so the framing is implemented from the specification:
//   greeting  64 bytes: FF 00*8 7F | 03 00 | "NULL" padded to 20 | as-server 00 | 31 x 00
//   handshake one READY command per side: 04 <len> 05 "READY" { <nlen> name <4-byte BE vlen> value }*
//   traffic   frames <flags> <size> <body>; flags bit0 MORE, bit1 LONG (8-byte BE size), bit2 COMMAND
//   REQ/REP   a request is [empty delimiter frame][body]; the reply repeats the envelope
//   PUSH/PULL messages are plain frame sequences
#pragma once
#include <errno.h>
#include <fcntl.h>
#include <poll.h>
#include <sys/socket.h>
#include <sys/stat.h>
#include <sys/un.h>
#include <unistd.h>

#include <chrono>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <memory>
#include <string>
#include <vector>

namespace zmtp {

enum SockType { REQ, REP, PUSH, PULL };
inline const char* type_name(SockType t) {
    switch (t) {
        case REQ: return "REQ";
        case REP: return "REP";
        case PUSH: return "PUSH";
        default: return "PULL";
    }
}
inline bool compatible(SockType local, const std::string& peer) {
    switch (local) {
        case REQ: return peer == "REP" || peer == "ROUTER";
        case REP: return peer == "REQ" || peer == "DEALER";
        case PUSH: return peer == "PULL";
        default: return peer == "PUSH";
    }
}

using Message = std::vector<std::string>;  // frames

inline std::string greeting() {
    std::string g(64, '\0');
    g[0] = (char)0xFF;
    g[9] = 0x7F;
    g[10] = 3;  // major
    g[11] = 0;  // minor
    std::memcpy(&g[12], "NULL", 4);
    return g;
}
inline void append_frame(std::string& out, const std::string& body, bool more, bool command) {
    uint8_t flags = (more ? 1 : 0) | (command ? 4 : 0);
    if (body.size() > 255) {
        out.push_back((char)(flags | 2));
        for (int s = 56; s >= 0; s -= 8) out.push_back((char)((uint64_t)body.size() >> s));
    } else {
        out.push_back((char)flags);
        out.push_back((char)body.size());
    }
    out.append(body);
}
inline std::string ready_command(SockType t) {
    std::string body;
    body.push_back(5);
    body.append("READY");
    auto prop = [&](const char* name, const std::string& value) {
        body.push_back((char)std::strlen(name));
        body.append(name);
        const uint32_t n = (uint32_t)value.size();
        body.push_back((char)(n >> 24));
        body.push_back((char)(n >> 16));
        body.push_back((char)(n >> 8));
        body.push_back((char)n);
        body.append(value);
    };
    prop("Socket-Type", type_name(t));
    if (t == REQ) prop("Identity", "");
    std::string out;
    append_frame(out, body, false, true);
    return out;
}

constexpr uint64_t kMaxFrame = 1ull << 31;

// One peer connection: incremental parser + blocking writer.
class Conn {
public:
    Conn(int fd, SockType local) : fd_(fd), local_(local) {
        int fl = fcntl(fd_, F_GETFL, 0);
        fcntl(fd_, F_SETFL, fl | O_NONBLOCK);
        send_raw(greeting() + ready_command(local_));
    }
    ~Conn() {
        if (fd_ >= 0) ::close(fd_);
    }
    Conn(const Conn&) = delete;
    Conn& operator=(const Conn&) = delete;

    int fd() const { return fd_; }
    uint64_t tag = 0;  // set by the owner: a name for this connection that is never reused
    bool failed() const { return failed_; }
    bool ready() const { return stage_ == 2; }
    const std::string& peer_type() const { return peer_type_; }
    std::deque<Message>& inbox() { return inbox_; }

    // Drains the socket and parses; false once the peer is gone or spoke nonsense.
    bool pump() {
        char buf[65536];
        for (;;) {
            const ssize_t n = ::recv(fd_, buf, sizeof(buf), 0);
            if (n > 0) {
                rbuf_.append(buf, (size_t)n);
                continue;
            }
            if (n == 0) {
                failed_ = true;
                break;
            }
            if (errno == EINTR) continue;
            if (errno != EAGAIN && errno != EWOULDBLOCK) failed_ = true;
            break;
        }
        parse();
        return !failed_ || !inbox_.empty();
    }

    bool send(const Message& m) {
        std::string out;
        for (size_t i = 0; i < m.size(); ++i) append_frame(out, m[i], i + 1 < m.size(), false);
        return send_raw(out);
    }

private:
    // The writer blocks, but not for ever: a peer that does not drain its socket for send_budget_ms()
    // in all while one message is written is dropped, so that one stalled reader cannot hold up a
    // single-threaded server and every other peer with it.
    static int send_budget_ms() {
        static const int ms = [] {
            const char* e = std::getenv("TORPOR_SEND_TIMEOUT_MS");
            const long v = (e && *e) ? std::strtol(e, nullptr, 10) : 0;
            return (int)(v > 0 && v < 3600000 ? v : 3000);
        }();
        return ms;
    }
    bool send_raw(const std::string& data) {
        size_t off = 0;
        if (failed_) return false;
        const auto deadline = std::chrono::steady_clock::now() + std::chrono::milliseconds(send_budget_ms());
        while (off < data.size()) {
            const ssize_t n = ::send(fd_, data.data() + off, data.size() - off, MSG_NOSIGNAL);
            if (n > 0) {
                off += (size_t)n;
                continue;
            }
            if (n < 0 && (errno == EAGAIN || errno == EWOULDBLOCK)) {
                const auto left = std::chrono::duration_cast<std::chrono::milliseconds>(
                                      deadline - std::chrono::steady_clock::now()).count();
                if (left <= 0) {
                    failed_ = true;
                    return false;
                }
                struct pollfd p = {fd_, POLLOUT, 0};
                ::poll(&p, 1, (int)(left < 1000 ? left : 1000));
                continue;
            }
            if (n < 0 && errno == EINTR) continue;
            failed_ = true;
            return false;
        }
        return true;
    }

    void parse() {
        size_t pos = 0;
        if (stage_ == 0) {
            if (rbuf_.size() < 64) return;
            const uint8_t* g = reinterpret_cast<const uint8_t*>(rbuf_.data());
            if (g[0] != 0xFF || g[9] != 0x7F || g[10] < 3 || std::memcmp(g + 12, "NULL\0", 5) != 0) {
                failed_ = true;
                return;
            }
            pos = 64;
            stage_ = 1;
        }
        for (;;) {
            if (rbuf_.size() - pos < 2) break;
            const uint8_t flags = (uint8_t)rbuf_[pos];
            uint64_t len = 0;
            size_t hdr = 2;
            if (flags & 2) {
                if (rbuf_.size() - pos < 9) break;
                for (int i = 0; i < 8; ++i) len = (len << 8) | (uint8_t)rbuf_[pos + 1 + i];
                hdr = 9;
            } else {
                len = (uint8_t)rbuf_[pos + 1];
            }
            // No legitimate message is larger than a protobuf message can be (2 GiB); the largest the
            // clients send is one weight tensor per upload.
            if (len > kMaxFrame) {
                failed_ = true;
                break;
            }
            if (rbuf_.size() - pos - hdr < len) break;
            std::string body = rbuf_.substr(pos + hdr, (size_t)len);
            pos += hdr + (size_t)len;
            if (flags & 4) {
                on_command(body);
            } else if (stage_ == 2) {
                partial_.push_back(std::move(body));
                if (!(flags & 1)) {
                    inbox_.push_back(std::move(partial_));
                    partial_.clear();
                }
            } else {
                failed_ = true;  // traffic before READY
            }
            if (failed_) break;
        }
        rbuf_.erase(0, pos);
    }

    void on_command(const std::string& body) {
        if (body.empty()) {
            failed_ = true;
            return;
        }
        const size_t nl = (uint8_t)body[0];
        if (body.size() < 1 + nl) {
            failed_ = true;
            return;
        }
        const std::string name = body.substr(1, nl);
        if (name == "READY") {
            size_t p = 1 + nl;
            while (p < body.size()) {
                const size_t kl = (uint8_t)body[p++];
                if (p + kl + 4 > body.size()) {
                    failed_ = true;
                    return;
                }
                const std::string key = body.substr(p, kl);
                p += kl;
                uint32_t vl = 0;
                for (int i = 0; i < 4; ++i) vl = (vl << 8) | (uint8_t)body[p + i];
                p += 4;
                if (p + vl > body.size()) {
                    failed_ = true;
                    return;
                }
                if (key == "Socket-Type") peer_type_ = body.substr(p, vl);
                p += vl;
            }
            if (!compatible(local_, peer_type_))
                failed_ = true;
            else
                stage_ = 2;
        } else if (name == "PING") {  // ZMTP 3.1 heartbeat: answer with PONG + context
            std::string pong;
            pong.push_back(4);
            pong.append("PONG");
            if (body.size() > 1 + nl + 2) pong.append(body.substr(1 + nl + 2));
            std::string out;
            append_frame(out, pong, false, true);
            send_raw(out);
        } else if (name == "ERROR") {
            failed_ = true;
        }
        // PONG / SUBSCRIBE / unknown commands are ignored
    }

    int fd_;
    SockType local_;
    int stage_ = 0;  // 0 greeting, 1 handshake, 2 traffic
    bool failed_ = false;
    std::string rbuf_, peer_type_;
    Message partial_;
    std::deque<Message> inbox_;
};

inline std::string ipc_path(const std::string& endpoint) {
    const std::string pre = "ipc://";
    return endpoint.compare(0, pre.size(), pre) == 0 ? endpoint.substr(pre.size()) : endpoint;
}

inline int listen_ipc(const std::string& endpoint) {
    const std::string path = ipc_path(endpoint);
    struct sockaddr_un addr;
    if (path.size() >= sizeof(addr.sun_path)) return -1;
    ::unlink(path.c_str());
    const int fd = ::socket(AF_UNIX, SOCK_STREAM, 0);
    if (fd < 0) return -1;
    std::memset(&addr, 0, sizeof(addr));
    addr.sun_family = AF_UNIX;
    std::strncpy(addr.sun_path, path.c_str(), sizeof(addr.sun_path) - 1);
    if (::bind(fd, reinterpret_cast<struct sockaddr*>(&addr), sizeof(addr)) != 0 || ::listen(fd, 128) != 0) {
        ::close(fd);
        return -1;
    }
    fcntl(fd, F_SETFL, fcntl(fd, F_GETFL, 0) | O_NONBLOCK);
    return fd;
}

inline int connect_ipc(const std::string& endpoint) {
    const std::string path = ipc_path(endpoint);
    struct sockaddr_un addr;
    if (path.size() >= sizeof(addr.sun_path)) return -1;
    const int fd = ::socket(AF_UNIX, SOCK_STREAM, 0);
    if (fd < 0) return -1;
    std::memset(&addr, 0, sizeof(addr));
    addr.sun_family = AF_UNIX;
    std::strncpy(addr.sun_path, path.c_str(), sizeof(addr.sun_path) - 1);
    if (::connect(fd, reinterpret_cast<struct sockaddr*>(&addr), sizeof(addr)) != 0) {
        ::close(fd);
        return -1;
    }
    return fd;
}

}  // namespace zmtp
