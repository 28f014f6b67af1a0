// server.cpp — poll loop, connection handling and packet dispatch of the token server
// (reference: server/server.cpp for the loop, server/client.cpp for the per-connection part).
#include "server.h"

#include <arpa/inet.h>
#include <csignal>
#include <cerrno>
#include <cstdio>
#include <cstring>
#include <iostream>
#include <netinet/in.h>
#include <poll.h>
#include <sys/eventfd.h>
#include <sys/signalfd.h>
#include <sys/socket.h>
#include <unistd.h>

#include "../ggml_file.h"
#include "../llava_context.h"
#include "session_wrapper.h"

namespace lsrv {

// One TCP connection: bytes received and not yet parsed, bytes queued and not yet sent.
struct llava_server::client {
    u32 id;
    int fd;
    std::vector<u8> input;
    std::vector<u8> output;
    size_t sent = 0;            // prefix of `output` already written to the socket
    bool overflowed = false;    // more output queued than a client may leave unread: dropped at the next write pass
    ~client() { if (fd >= 0) ::close(fd); }
};

llava_server::llava_server(llava_context *context, u16 _port, std::string _bind_address)
    : ctx(context), port(_port), bind_address(std::move(_bind_address))
{
    // the vocabulary never changes: build the cmdGetTokenMap answer once (server/server.cpp:29-42)
    if (const ggml_file *model = ctx->get_model())
        for (const ggml_token &token : model->get_tokens()) {
            put_u32(token_map_payload, static_cast<u32>(token.text.size()));
            token_map_payload.insert(token_map_payload.end(), token.text.begin(), token.text.end());
        }
}

llava_server::~llava_server()
{
    stop_sessions();
    for (auto &entry : sessions) entry.second->join();
    sessions.clear();
    clients.clear();
    for (int fd : {listen_fd, wake_fd, signal_fd})
        if (fd >= 0) ::close(fd);
}

bool llava_server::open()
{
    if (listen_fd >= 0) return true;
    wake_fd = eventfd(0, EFD_NONBLOCK | EFD_CLOEXEC);
    if (wake_fd < 0) {
        std::perror("eventfd");
        return false;
    }
    const int s = socket(AF_INET, SOCK_STREAM | SOCK_CLOEXEC, 0);
    if (s < 0) {
        std::perror("socket");
        return false;
    }
    const int enable = 1;
    sockaddr_in addr{};
    addr.sin_family = AF_INET;
    addr.sin_port = htons(port);
    socklen_t len = sizeof addr;
    if (setsockopt(s, SOL_SOCKET, SO_REUSEADDR, &enable, sizeof enable) < 0 || inet_pton(AF_INET, bind_address.c_str(), &addr.sin_addr) != 1 ||
        bind(s, reinterpret_cast<sockaddr *>(&addr), sizeof addr) < 0 || listen(s, 16) < 0 ||
        getsockname(s, reinterpret_cast<sockaddr *>(&addr), &len) < 0) {
        std::cerr << "[!] cannot listen on " << bind_address << ":" << port << ": " << std::strerror(errno) << std::endl;
        ::close(s);
        return false;
    }
    port = ntohs(addr.sin_port);
    listen_fd = s;
    return true;
}

void llava_server::wake()
{
    const uint64_t one = 1;
    if (wake_fd >= 0 && ::write(wake_fd, &one, sizeof one) != static_cast<ssize_t>(sizeof one) && errno != EAGAIN)
        std::cerr << "[?] wake-up of the poll loop failed: " << std::strerror(errno) << std::endl;
}

void llava_server::block_termination_signals()
{
    sigset_t mask;
    sigemptyset(&mask);
    for (int sig : {SIGINT, SIGQUIT, SIGHUP, SIGTERM}) sigaddset(&mask, sig);
    pthread_sigmask(SIG_BLOCK, &mask, nullptr);
}

void llava_server::request_stop()
{
    stop_requested.store(true);
    wake();
}

void llava_server::post(std::vector<outbound_message> &messages)
{
    {
        std::lock_guard<std::mutex> lock(posted_mutex);
        for (outbound_message &m : messages) posted.push_back(std::move(m));
    }
    messages.clear();
    wake();
}

void llava_server::notify_session_death(u32 session_id)
{
    {
        std::lock_guard<std::mutex> lock(posted_mutex);
        dead_sessions.push_back(session_id);
    }
    wake();
}

void llava_server::send_to(client &c, OutCommands kind, u32 reply_to, const std::vector<u8> &payload)
{
    if (c.overflowed) return;
    if (c.output.size() - c.sent + sizeof(tlv_header) + payload.size() > kMaxOutputBuffer) {
        std::cerr << "[!] client " << c.id << " does not read its replies, dropping it" << std::endl;
        c.overflowed = true;
        return;
    }
    put_u32(c.output, kind);
    put_u32(c.output, reply_to);
    put_u32(c.output, static_cast<u32>(payload.size()));
    c.output.insert(c.output.end(), payload.begin(), payload.end());
}

void llava_server::ack(client &c, u32 request_id, ReturnCode code) { send_to(c, outCmdAck, request_id, words({static_cast<u32>(code)})); }

void llava_server::accept_client()
{
    sockaddr_in peer{};
    socklen_t len = sizeof peer;
    const int fd = accept4(listen_fd, reinterpret_cast<sockaddr *>(&peer), &len, SOCK_NONBLOCK | SOCK_CLOEXEC);
    if (fd < 0) {
        if (errno != EAGAIN && errno != EINTR) std::perror("accept");
        return;
    }
    char text[INET_ADDRSTRLEN] = "?";
    inet_ntop(AF_INET, &peer.sin_addr, text, sizeof text);
    auto c = std::make_unique<client>();
    c->id = next_client_id++;
    c->fd = fd;
    std::cout << "[*] client " << c->id << " from " << text << ":" << ntohs(peer.sin_port) << std::endl;
    clients.emplace(c->id, std::move(c));
}

// Every client learns of a new session; the one that asked gets its request id back (server/server.cpp:256-263).
void llava_server::create_session(client &caller, u32 request_id)
{
    const u32 id = next_session_id++;
    auto wrapper = std::make_unique<session_wrapper>(this, id);
    for (auto &entry : clients) send_to(*entry.second, outCmdNewSession, entry.second.get() == &caller ? request_id : 0, words({id}));
    wrapper->start();
    sessions.emplace(id, std::move(wrapper));
}

void llava_server::handle_packet(client &c, const tlv_header &h, const u8 *body)
{
    auto session_of = [&](u32 id) -> session_wrapper * {
        auto it = sessions.find(id);
        return it == sessions.end() ? nullptr : it->second.get();
    };
    if (h.command < 16) {
        switch (h.command) {
        case cmdGetTokenMap: send_to(c, outCmdTokenMap, h.request_id, token_map_payload); break;
        case cmdNewSession: create_session(c, h.request_id); break;
        case cmdListSessions: {
            std::vector<u8> ids;
            for (const auto &entry : sessions) put_u32(ids, entry.first);
            send_to(c, outCmdSessionList, h.request_id, ids);
            break;
        }
        default: ack(c, h.request_id, ReturnCode::unknown_command);
        }
        return;
    }
    // every other command starts with the session it is for
    const bool with_value = h.command == cmdRewind || h.command == cmdAddToken || h.command == cmdSetSessionOptions;
    const bool with_text = h.command == cmdAddText || h.command == cmdSaveFrame || h.command == cmdSnapshot || h.command == cmdRestore;
    if (h.command >= 32 && !with_value && !with_text) return ack(c, h.request_id, ReturnCode::unknown_command);
    const bool length_ok = with_text ? h.length > 4 : h.length == (with_value ? 8u : 4u);
    if (!length_ok) return ack(c, h.request_id, ReturnCode::bad_arguments);
    const u32 session_id = get_u32(body);
    session_wrapper *session = session_of(session_id);
    if (!session) return ack(c, h.request_id, ReturnCode::no_such_session);

    if (with_value) return session->push_order(c.id, h.request_id, h.command, get_u32(body + 4));
    if (with_text) {
        std::string text(reinterpret_cast<const char *>(body + 4), h.length - 4);
        const size_t nul = text.find('\0');
        if (nul != std::string::npos) {
            // a path with a NUL in it is refused; text is cut there, as the reference's C-string copy does
            if (h.command != cmdAddText) return ack(c, h.request_id, ReturnCode::bad_arguments);
            std::cerr << "[?] NUL byte in added text" << std::endl;
            text.resize(nul);
        }
        return session->push_order(c.id, h.request_id, h.command, 0, std::move(text));
    }
    switch (h.command) {
    case cmdSubscribe:
        subscribers[session_id].insert(c.id);
        return ack(c, h.request_id, ReturnCode::ok);
    case cmdUnsubscribe:
        subscribers[session_id].erase(c.id);
        return ack(c, h.request_id, ReturnCode::ok);
    case cmdGetSessionTokens:
    case cmdKillSession:
    case cmdStartSessionGeneration:
    case cmdStopSessionGeneration:
    case cmdTick:
    case cmdGetSessionStatus:
        return session->push_order(c.id, h.request_id, h.command);
    default:
        return ack(c, h.request_id, ReturnCode::unknown_command);
    }
}

bool llava_server::service_client(client &c, short revents)
{
    if (revents & (POLLERR | POLLHUP | POLLNVAL)) return false;
    if (revents & POLLIN) {
        u8 chunk[4096];
        while (c.input.size() < kMaxInputBuffer) {
            const ssize_t n = recv(c.fd, chunk, sizeof chunk, 0);
            if (n > 0) {
                c.input.insert(c.input.end(), chunk, chunk + n);
                if (static_cast<size_t>(n) < sizeof chunk) break;
            } else if (n == 0) {
                return false;           // orderly shutdown by the peer
            } else if (errno == EAGAIN || errno == EWOULDBLOCK) {
                break;
            } else if (errno != EINTR) {
                std::perror("recv");
                return false;
            }
        }
        size_t at = 0;
        while (c.input.size() - at >= sizeof(tlv_header)) {
            const u8 *p = c.input.data() + at;
            const tlv_header h = {get_u32(p), get_u32(p + 4), get_u32(p + 8)};
            if (h.length > kMaxPacketLength) {
                // the reference stops parsing such a client and keeps its socket (server/client.cpp:129-133); unread input
                // would then keep the poll loop spinning, so the connection is closed instead
                std::cerr << "[!] client " << c.id << ": packet of " << h.length << " bytes, closing the connection" << std::endl;
                return false;
            }
            if (c.input.size() - at < sizeof(tlv_header) + h.length) break;
            handle_packet(c, h, p + sizeof(tlv_header));
            at += sizeof(tlv_header) + h.length;
        }
        c.input.erase(c.input.begin(), c.input.begin() + static_cast<std::ptrdiff_t>(at));
    }
    return true;
}

// packets the session threads queued: to one client, or to the subscribers of the session
void llava_server::deliver_posted()
{
    std::vector<outbound_message> batch;
    {
        std::lock_guard<std::mutex> lock(posted_mutex);
        batch.swap(posted);
    }
    for (const outbound_message &m : batch) {
        if (m.client_id) {
            auto it = clients.find(m.client_id);
            if (it != clients.end()) send_to(*it->second, m.kind, m.reply_to, m.payload);
            continue;
        }
        auto subs = subscribers.find(m.session);
        if (subs == subscribers.end()) continue;
        for (u32 client_id : subs->second) {
            auto it = clients.find(client_id);
            if (it != clients.end()) send_to(*it->second, m.kind, m.reply_to, m.payload);
        }
    }
}

void llava_server::reap_sessions()
{
    std::vector<u32> dead;
    {
        std::lock_guard<std::mutex> lock(posted_mutex);
        dead.swap(dead_sessions);
    }
    for (u32 id : dead) {
        auto it = sessions.find(id);
        if (it == sessions.end()) continue;
        it->second->join();
        sessions.erase(it);
        subscribers.erase(id);
        for (auto &entry : clients) send_to(*entry.second, outCmdDroppedSession, 0, words({id}));
    }
}

void llava_server::drop_client(u32 client_id)
{
    for (auto &entry : subscribers) entry.second.erase(client_id);
    clients.erase(client_id);
}

void llava_server::stop_sessions()
{
    for (auto &entry : sessions) entry.second->push_order(0, 0, cmdKillSession);
}

bool llava_server::serve_forever()
{
    if (!open()) return false;
    // termination signals arrive through a descriptor, like every other event of the loop
    block_termination_signals();
    sigset_t mask;
    sigemptyset(&mask);
    for (int sig : {SIGINT, SIGQUIT, SIGHUP, SIGTERM}) sigaddset(&mask, sig);
    signal_fd = signalfd(-1, &mask, SFD_NONBLOCK | SFD_CLOEXEC);
    const bool watch_stdin = isatty(STDIN_FILENO) != 0;   // a key press ends the server; a closed or redirected stdin does not
    std::cout << "[*] Started server on " << bind_address << ":" << port << std::endl;

    bool stopping = false;
    std::vector<pollfd> fds;
    std::vector<u32> polled_clients;
    while (!stopping || !sessions.empty()) {
        fds.clear();
        polled_clients.clear();
        fds.push_back({wake_fd, POLLIN, 0});
        fds.push_back({stopping ? -1 : listen_fd, POLLIN, 0});
        fds.push_back({signal_fd, POLLIN, 0});                       // a negative descriptor is skipped by poll
        fds.push_back({watch_stdin && !stopping ? STDIN_FILENO : -1, POLLIN, 0});
        for (auto &entry : clients) {
            client &c = *entry.second;
            const short events = static_cast<short>(POLLIN | (c.sent < c.output.size() ? POLLOUT : 0));
            fds.push_back({c.fd, events, 0});
            polled_clients.push_back(c.id);
        }
        const int ready = poll(fds.data(), fds.size(), 1000);
        if (ready < 0) {
            if (errno == EINTR) continue;
            std::cerr << "[?] poll: " << std::strerror(errno) << std::endl;
            break;
        }
        if (fds[0].revents & POLLIN) {
            uint64_t count;
            while (::read(wake_fd, &count, sizeof count) == static_cast<ssize_t>(sizeof count)) {}
        }
        if (fds[2].revents & POLLIN) {
            signalfd_siginfo info;
            while (::read(signal_fd, &info, sizeof info) == static_cast<ssize_t>(sizeof info)) {}
            stop_requested.store(true);
        }
        if (fds[3].revents & (POLLIN | POLLHUP)) stop_requested.store(true);
        if (stop_requested.load() && !stopping) {
            stopping = true;
            stop_sessions();
        }
        if (fds[1].revents & POLLIN) accept_client();

        std::vector<u32> to_drop;
        for (size_t i = 0; i < polled_clients.size(); ++i) {
            auto it = clients.find(polled_clients[i]);
            if (it == clients.end()) continue;
            if (fds[4 + i].revents && !service_client(*it->second, fds[4 + i].revents)) to_drop.push_back(it->first);
        }
        for (u32 id : to_drop) drop_client(id);

        deliver_posted();
        reap_sessions();

        // write what is queued; whatever the socket does not take now waits for POLLOUT
        to_drop.clear();
        for (auto &entry : clients) {
            client &c = *entry.second;
            if (c.overflowed) {
                to_drop.push_back(c.id);
                continue;
            }
            while (c.sent < c.output.size()) {
                const ssize_t n = send(c.fd, c.output.data() + c.sent, c.output.size() - c.sent, MSG_NOSIGNAL);
                if (n > 0) {
                    c.sent += static_cast<size_t>(n);
                } else if (n < 0 && (errno == EAGAIN || errno == EWOULDBLOCK)) {
                    break;
                } else if (n < 0 && errno == EINTR) {
                    continue;
                } else {
                    to_drop.push_back(c.id);
                    break;
                }
            }
            if (c.sent == c.output.size()) {
                c.output.clear();
                c.sent = 0;
            }
        }
        for (u32 id : to_drop) drop_client(id);
    }
    clients.clear();
    ::close(listen_fd);
    listen_fd = -1;
    return true;
}

}  // namespace lsrv
