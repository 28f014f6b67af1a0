// session_wrapper.h — one llava_session living on its own thread, driven by orders from the server's poll loop
// (reference: server/session_wrapper.h).  The thread starts a step, handles whatever orders arrived while the
// device works, and only then waits for the token: the overlap start/finish are split for.
#pragma once

#include <condition_variable>
#include <deque>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "protocol.h"

class llava_session;

namespace lsrv {

class llava_server;

class session_wrapper {
public:
    session_wrapper(llava_server *server, u32 session_id);
    ~session_wrapper();             // joins the thread; send cmdKillSession first or this blocks
    session_wrapper(const session_wrapper &) = delete;
    session_wrapper &operator=(const session_wrapper &) = delete;

    void start();
    // any thread
    void push_order(u32 client_id, u32 request_id, u32 opcode, u32 arg1 = 0, std::string s = {});
    void join();

    const u32 session_id;
    llava_server *const server;

private:
    void run();
    // handles every queued order; with `blocking` it first sleeps until there is one
    void process_orders(llava_session &session, bool blocking);
    ReturnCode execute(llava_session &session, const session_order &order, bool &acknowledge);
    void produce_token(llava_session &session);
    void reply(u32 client_id, OutCommands kind, u32 reply_to, std::vector<u8> payload);
    void ack(u32 client_id, u32 request_id, ReturnCode code);
    void flush();

    std::mutex order_mutex;
    std::condition_variable order_arrived;
    std::deque<session_order> orders;
    std::thread worker;

    // state of the session thread only
    std::vector<outbound_message> outbox;
    bool generating = false;    // cmdStartSessionGeneration .. cmdStopSessionGeneration
    u32 tick_request = 0;       // request id of a pending cmdTick, 0 = none
    u32 tick_client = 0;
    bool dying = false;
    bool greedy = false;
};

}  // namespace lsrv
