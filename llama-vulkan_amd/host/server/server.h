// server.h — the token server: one poll loop owning the listening socket, the clients and the table of sessions;
// every session runs on a thread of its own (session_wrapper) and posts its packets back through a queue and an
// eventfd (reference: server/server.h, server/client.h).
#pragma once

#include <atomic>
#include <map>
#include <memory>
#include <mutex>
#include <set>
#include <string>
#include <vector>

#include "protocol.h"

class llava_context;

namespace lsrv {

class session_wrapper;

class llava_server {
public:
    // port 0 asks the system for a free one (see bound_port()).  The reference listens on 0.0.0.0:1337.
    explicit llava_server(llava_context *context, u16 port = 1337, std::string bind_address = "0.0.0.0");
    ~llava_server();
    llava_server(const llava_server &) = delete;
    llava_server &operator=(const llava_server &) = delete;

    // Binds and listens; false + message on stderr when that fails.  Separate from serve_forever() so that a
    // caller can learn the port before the loop starts.
    bool open();
    // Runs until a termination signal, input on a terminal's stdin, or request_stop(); then kills the sessions,
    // waits for them and closes every connection.  Calls open() when that was not done.
    bool serve_forever();
    void request_stop();                        // any thread
    // Blocks SIGINT, SIGQUIT, SIGHUP and SIGTERM for the calling thread and every thread it creates afterwards, so
    // that they reach serve_forever() through its signalfd.  A process must call this before anything starts a
    // thread (the device runtime does): a signal goes to any thread that has not blocked it.
    static void block_termination_signals();
    [[nodiscard]] u16 bound_port() const { return port; }

    // ---- called by session threads ----------------------------------------------------------------------
    void post(std::vector<outbound_message> &messages);     // takes the messages
    void notify_session_death(u32 session_id);

    llava_context *const ctx;

private:
    struct client;
    void wake();
    void accept_client();
    bool service_client(client &c, short revents);          // false: drop the client
    void handle_packet(client &c, const tlv_header &header, const u8 *body);
    void send_to(client &c, OutCommands kind, u32 reply_to, const std::vector<u8> &payload);
    void ack(client &c, u32 request_id, ReturnCode code);
    void create_session(client &caller, u32 request_id);
    void deliver_posted();
    void reap_sessions();
    void drop_client(u32 client_id);
    void stop_sessions();

    u16 port;
    const std::string bind_address;
    int listen_fd = -1, wake_fd = -1, signal_fd = -1;
    std::atomic<bool> stop_requested{false};
    std::vector<u8> token_map_payload;

    // poll-loop state
    std::map<u32, std::unique_ptr<client>> clients;                 // by client id
    std::map<u32, std::unique_ptr<session_wrapper>> sessions;       // by session id
    std::map<u32, std::set<u32>> subscribers;                       // session id -> client ids
    u32 next_client_id = 1, next_session_id = 1;

    // filled by session threads
    std::mutex posted_mutex;
    std::vector<outbound_message> posted;
    std::vector<u32> dead_sessions;
};

}  // namespace lsrv
