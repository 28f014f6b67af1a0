"""A client of the token server's wire protocol for the tests, written from the packet layout alone (little-endian
u32 command, u32 request id, u32 length, arguments; answers come back as u32 kind, u32 reply_to, u32 length, payload;
reference: server/types.h:50-115), independently of the C++ that implements the server side."""
import socket
import struct

GET_TOKEN_MAP, NEW_SESSION, LIST_SESSIONS = 0, 1, 2
GET_TOKENS, SUBSCRIBE, UNSUBSCRIBE, KILL, START, STOP, TICK, STATUS = 16, 17, 18, 19, 20, 21, 22, 23
REWIND, ADD_TOKEN, ADD_TEXT, SET_OPTIONS, SAVE_FRAME, SNAPSHOT, RESTORE = 32, 33, 34, 35, 36, 37, 38
OUT_TOKEN, OUT_BUFFER, OUT_TOKEN_MAP, OUT_NEW_SESSION, OUT_SESSION_LIST, OUT_DROPPED, OUT_ACK, OUT_STATUS = range(8)
RC_OK, RC_NOK, RC_NO_SUCH_SESSION, RC_TICK_PENDING, RC_RUNNING, RC_NOT_TRACING, RC_BATCHED, RC_BAD_ARGS, RC_UNKNOWN = range(9)
OPTION_RECORD, OPTION_GREEDY = 1, 2


class Client:
    def __init__(self, port, timeout=20.0):
        self.sock = socket.create_connection(("127.0.0.1", port), timeout=timeout)
        self.buf = b""
        self.next_id = 1
        self.unsolicited = []       # packets with reply_to 0, in arrival order: (kind, payload)

    def close(self):
        self.sock.close()

    def send_raw(self, data):
        self.sock.sendall(data)

    def request(self, command, body=b""):
        rid = self.next_id
        self.next_id += 1
        self.sock.sendall(struct.pack("<3I", command, rid, len(body)) + body)
        return rid

    def read_packet(self):
        while True:
            if len(self.buf) >= 12:
                kind, reply_to, length = struct.unpack_from("<3I", self.buf)
                if len(self.buf) >= 12 + length:
                    payload = self.buf[12:12 + length]
                    self.buf = self.buf[12 + length:]
                    return kind, reply_to, payload
            chunk = self.sock.recv(65536)
            if not chunk:
                raise ConnectionError("the server closed the connection")
            self.buf += chunk

    def wait_reply(self, rid):
        """the packet answering request `rid`; everything unasked-for that arrives before it is kept"""
        while True:
            kind, reply_to, payload = self.read_packet()
            if reply_to == rid:
                return kind, payload
            assert reply_to == 0, (kind, reply_to)
            self.unsolicited.append((kind, payload))

    def wait_unsolicited(self, kind):
        while True:
            for i, (k, payload) in enumerate(self.unsolicited):
                if k == kind:
                    del self.unsolicited[i]
                    return payload
            k, reply_to, payload = self.read_packet()
            assert reply_to == 0, (k, reply_to)
            self.unsolicited.append((k, payload))

    def call(self, command, body=b""):
        return self.wait_reply(self.request(command, body))

    def ack(self, command, *words, text=b""):
        """sends a command whose answer is an acknowledgement and returns its return code"""
        kind, payload = self.call(command, struct.pack(f"<{len(words)}I", *words) + text)
        assert kind == OUT_ACK and len(payload) == 4, (kind, payload)
        return struct.unpack("<I", payload)[0]

    def new_session(self):
        kind, payload = self.call(NEW_SESSION)
        assert kind == OUT_NEW_SESSION
        return struct.unpack("<I", payload)[0]

    def sessions(self):
        kind, payload = self.call(LIST_SESSIONS)
        assert kind == OUT_SESSION_LIST
        return list(struct.unpack(f"<{len(payload) // 4}I", payload))

    def tokens(self, session):
        kind, payload = self.call(GET_TOKENS, struct.pack("<I", session))
        assert kind == OUT_BUFFER
        return list(struct.unpack(f"<{len(payload) // 4}I", payload))

    def tick(self, session):
        """one token: (token, index) on success, the return code otherwise"""
        kind, payload = self.call(TICK, struct.pack("<I", session))
        if kind == OUT_ACK:
            return struct.unpack("<I", payload)[0]
        assert kind == OUT_TOKEN
        sid, token, index = struct.unpack("<3I", payload)
        assert sid == session
        return token, index
