// Small host utilities: error reporting, sha256, file IO.
#pragma once
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

namespace iu8 {

// The calling thread's last error message and code.
void set_error(int code, const std::string &msg);
int fail(int code, const std::string &msg);  // records and returns `code`
const char *last_error();

bool read_file(const std::string &path, std::vector<uint8_t> &out);
bool write_file(const std::string &path, const std::string &text);

std::string sha256_hex(const uint8_t *data, size_t len);
void sha256(const uint8_t *data, size_t len, uint8_t out[32]);

std::string fmt(const char *f, ...) __attribute__((format(printf, 1, 2)));

}  // namespace iu8
