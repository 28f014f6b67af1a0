// session_wrapper.cpp — the session thread of the token server (reference: server/session_wrapper.cpp).
#include "session_wrapper.h"

#include <csignal>
#include <iostream>
#include <utility>

#include "../llava_context.h"
#include "../llava_session.h"
#include "server.h"

namespace lsrv {

session_wrapper::session_wrapper(llava_server *_server, u32 _session_id) : session_id(_session_id), server(_server) {}

session_wrapper::~session_wrapper() { join(); }

void session_wrapper::start()
{
    if (!worker.joinable()) worker = std::thread([this] { run(); });
}

void session_wrapper::join()
{
    if (worker.joinable()) worker.join();
}

void session_wrapper::push_order(u32 client_id, u32 request_id, u32 opcode, u32 arg1, std::string s)
{
    {
        std::lock_guard<std::mutex> lock(order_mutex);
        orders.push_back({client_id, request_id, opcode, arg1, std::move(s)});
    }
    order_arrived.notify_one();
}

void session_wrapper::reply(u32 client_id, OutCommands kind, u32 reply_to, std::vector<u8> payload)
{
    outbox.push_back({client_id, session_id, kind, reply_to, std::move(payload)});
}

void session_wrapper::ack(u32 client_id, u32 request_id, ReturnCode code)
{
    // orders the server itself issues (shutdown) carry no client and are not answered
    if (client_id && request_id) reply(client_id, outCmdAck, request_id, words({static_cast<u32>(code)}));
}

void session_wrapper::flush()
{
    if (!outbox.empty()) server->post(outbox);     // takes the messages, leaves the vector empty
}

void session_wrapper::run()
{
    // termination signals belong to the poll loop's signalfd (server/session_wrapper.cpp:104-115)
    sigset_t mask;
    sigemptyset(&mask);
    for (int sig : {SIGINT, SIGQUIT, SIGHUP, SIGTERM}) sigaddset(&mask, sig);
    pthread_sigmask(SIG_BLOCK, &mask, nullptr);

    llava_session session(server->ctx);
    if (!session.good()) std::cerr << "[!] session " << session_id << " has no device session: every step will be refused" << std::endl;
    while (!dying) {
        process_orders(session, !(generating || tick_request));
        if (dying) break;
        if (generating || tick_request) produce_token(session);
    }
    process_orders(session, false);     // answer what arrived after the kill
    server->notify_session_death(session_id);
}

// One token: submit, serve orders while the device works, wait, publish (server/session_wrapper.cpp:58-97).
void session_wrapper::produce_token(llava_session &session)
{
    auto fail = [&](const char *what) {
        std::cerr << "[!] session " << session_id << ": " << what << std::endl;
        generating = false;
        if (tick_request) ack(tick_client, tick_request, ReturnCode::nok);
        tick_request = tick_client = 0;
        flush();
    };
    if (!session.good() || !session.start_next_token_prediction()) return fail("cannot start a step");
    const u32 tick_now = tick_request, tick_for = tick_client;
    process_orders(session, false);
    const u32 token = session.finish_next_token_prediction(greedy);
    if (token == ~0u) return fail("the device reported an error");
    const u32 index = session.get_token_count();
    std::vector<u8> packet = words({session_id, token, index});
    if (!session.push_token(token)) {
        std::cerr << "[*] session " << session_id << ": context full, generation stops" << std::endl;
        generating = false;
    }
    reply(0, outCmdNewToken, 0, packet);                                     // to the subscribers
    if (tick_now) reply(tick_for, outCmdNewToken, tick_now, std::move(packet));
    tick_request = tick_client = 0;
    flush();
}

void session_wrapper::process_orders(llava_session &session, bool blocking)
{
    std::deque<session_order> batch;
    {
        std::unique_lock<std::mutex> lock(order_mutex);
        if (blocking) order_arrived.wait(lock, [this] { return !orders.empty(); });
        batch.swap(orders);
    }
    for (const session_order &order : batch) {
        bool acknowledge = true;
        const ReturnCode code = execute(session, order, acknowledge);
        if (acknowledge) ack(order.client_id, order.request_id, code);
    }
    flush();
}

ReturnCode session_wrapper::execute(llava_session &session, const session_order &order, bool &acknowledge)
{
    switch (order.opcode) {
    case cmdStartSessionGeneration:
        if (tick_request) return ReturnCode::tick_already_requested;
        generating = true;
        return ReturnCode::ok;
    case cmdStopSessionGeneration:
        generating = false;
        return ReturnCode::ok;
    case cmdTick:
        if (generating) return ReturnCode::already_running;
        if (tick_request) return ReturnCode::tick_already_requested;
        tick_request = order.request_id;
        tick_client = order.client_id;
        acknowledge = false;            // the token is the answer
        return ReturnCode::ok;
    case cmdKillSession:
        dying = true;
        return ReturnCode::ok;
    case cmdRewind:
        session.rewind(order.arg1);
        return ReturnCode::ok;
    case cmdSetSessionOptions:
        greedy = (order.arg1 & kOptionGreedy) != 0;
        return session.set_options(order.arg1 & ~kOptionGreedy);
    case cmdAddToken:
        return session.push_token(order.arg1) ? ReturnCode::ok : ReturnCode::nok;
    case cmdAddText:
        return session.add_text(order.s) ? ReturnCode::ok : ReturnCode::nok;
    case cmdGetSessionTokens: {
        acknowledge = false;
        std::vector<u8> payload;
        payload.reserve(4 * session.get_token_buffer().size());
        for (u32 t : session.get_token_buffer()) put_u32(payload, t);
        reply(order.client_id, outCmdBuffer, order.request_id, std::move(payload));
        return ReturnCode::ok;
    }
    case cmdSaveFrame:
        return session.save_frame(order.s);
    case cmdSnapshot:
        return session.snapshot(order.s);
    case cmdRestore:
        if (generating) return ReturnCode::already_running;
        if (tick_request) return ReturnCode::tick_already_requested;
        return session.restore(order.s);
    default:
        return ReturnCode::ok;          // cmdGetSessionStatus and anything newer: acknowledged, as the reference does
    }
}

}  // namespace lsrv
