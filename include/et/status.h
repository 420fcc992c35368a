// Error policy of the C++ class layer: a failed C-ABI call throws et::Error
// (the reference asserts and exits, lib/utils.cu:28-35; an uncaught et::Error
// ends the process the same way, a caller may also catch it).
#pragma once
#include <stdexcept>
#include <string>

#include "../et_abi.h"

namespace et {

class Error : public std::runtime_error {
  public:
    Error(int status, const std::string &what) : std::runtime_error(what), status_(status) {}
    int status() const { return status_; }

  private:
    int status_;
};

inline void chk(int status, const char *file, int line) {
    if (status == ET_OK) return;
    throw Error(status, std::string(file) + ":" + std::to_string(line) + ": " +
                            et_status_string(status) + " — " + et_last_error());
}

inline void require(bool cond, const char *msg) {
    if (!cond) throw Error(ET_ERR_INVALID_ARG, msg);
}

using stream_t = et_stream;

}  // namespace et

#define etChk(stat) ::et::chk((stat), __FILE__, __LINE__)
