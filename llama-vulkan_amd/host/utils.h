// utils.h — small helpers shared by the host classes (reference: utils.h / utils.cpp).
#pragma once

#include <cstddef>
#include <string>

#include "types.h"

// printable name of an element type, nullptr for ids outside the enum (utils.cpp:6-38)
const char *ftype_name(ggml_value_type type);

// ceil(a / b) (utils.h:9-11)
inline u64 updiv(u64 a, u64 b) { return (a + b - 1) / b; }

// log2 of a power of two; 0xFFFFFFFF for anything else (the reference asserts instead, utils.cpp:52-61)
u32 ulog2(u32 n);

bool starts_with(const std::string &text, const std::string &prefix);
bool ends_with(const std::string &text, const std::string &suffix);

// read()/write() until everything moved or the descriptor gives up; return the byte count done (utils.cpp:63-90)
std::size_t read_noshort(int fd, void *dst, std::size_t size);
std::size_t write_noshort(int fd, const void *src, std::size_t size);
