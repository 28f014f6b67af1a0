// protocol.h — the wire format of the token server: little-endian TLV packets over one TCP stream per client.
// Command and reply numbers follow the reference (server/types.h:50-115) so that its clients keep working.
//
//   client -> server:  u32 command, u32 request_id, u32 length, length bytes of arguments
//   server -> client:  u32 kind,    u32 reply_to,   u32 length, length bytes of payload
//
// reply_to repeats the request_id of the packet being answered; 0 marks a packet nobody asked for (a token of a
// subscribed session, the announcement of a session another client created).
#pragma once

#include <cstring>
#include <string>
#include <vector>

#include "../types.h"

namespace lsrv {

enum Commands : u32 {
    // no arguments
    cmdGetTokenMap = 0,             // -> outCmdTokenMap
    cmdNewSession = 1,              // -> outCmdNewSession, to every client
    cmdListSessions = 2,            // -> outCmdSessionList
    // arguments: u32 session
    cmdGetSessionTokens = 16,       // -> outCmdBuffer
    cmdSubscribe = 17,              // this client receives the session's tokens from now on
    cmdUnsubscribe = 18,
    cmdKillSession = 19,
    cmdStartSessionGeneration = 20, // the session produces tokens until stopped or full
    cmdStopSessionGeneration = 21,
    cmdTick = 22,                   // one token; answered by outCmdNewToken instead of an ack
    cmdGetSessionStatus = 23,
    // arguments: u32 session, u32 value
    cmdRewind = 32,
    cmdAddToken = 33,
    cmdSetSessionOptions = 35,
    // arguments: u32 session, then text without a terminator
    cmdAddText = 34,
    cmdSaveFrame = 36,
    cmdSnapshot = 37,
    cmdRestore = 38,
};

enum OutCommands : u32 {
    outCmdNewToken = 0,         // u32 session, u32 token, u32 index of the token in the session's buffer
    outCmdBuffer = 1,           // u32 tokens[]
    outCmdTokenMap = 2,         // per vocabulary entry: u32 length, bytes
    outCmdNewSession = 3,       // u32 session
    outCmdSessionList = 4,      // u32 sessions[]
    outCmdDroppedSession = 5,   // u32 session
    outCmdAck = 6,              // u32 ReturnCode
    outCmdSessionStatus = 7,
};

// session option bits of cmdSetSessionOptions.  The reference knows record mode only (any non-zero value);
// the greedy bit is an addition: its sampler is always the stochastic one.
constexpr u32 kOptionRecord = 1u;
constexpr u32 kOptionGreedy = 2u;

struct tlv_header {
    u32 command, request_id, length;
};
static_assert(sizeof(tlv_header) == 12, "three packed words");

constexpr u32 kMaxPacketLength = 0x10000;   // a longer packet ends the connection (the reference marks the client failed: server/client.cpp:129-133)
constexpr u32 kMaxInputBuffer = 0x20000;    // unread input kept per client
constexpr u32 kMaxOutputBuffer = 16u << 20; // replies a client may leave unread before it is dropped

inline void put_u32(std::vector<u8> &out, u32 v)
{
    const u8 b[4] = {static_cast<u8>(v), static_cast<u8>(v >> 8), static_cast<u8>(v >> 16), static_cast<u8>(v >> 24)};
    out.insert(out.end(), b, b + 4);
}

inline u32 get_u32(const u8 *p) { return static_cast<u32>(p[0]) | static_cast<u32>(p[1]) << 8 | static_cast<u32>(p[2]) << 16 | static_cast<u32>(p[3]) << 24; }

inline std::vector<u8> words(std::initializer_list<u32> values)
{
    std::vector<u8> out;
    out.reserve(4 * values.size());
    for (u32 v : values) put_u32(out, v);
    return out;
}

// one packet from the server, and who gets it: client_id != 0 names one client; client_id == 0 sends it to
// every subscriber of `session`
struct outbound_message {
    u32 client_id;
    u32 session;
    OutCommands kind;
    u32 reply_to;
    std::vector<u8> payload;
};

// what a session thread is asked to do (server/types.h:16-22)
struct session_order {
    u32 client_id;
    u32 request_id;
    u32 opcode;
    u32 arg1;
    std::string s;
};

}  // namespace lsrv
