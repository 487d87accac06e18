// Thread-local error text of the host library's C entry points (bt_encoder_last_error).
#pragma once
#include <string>

namespace bt_host {
__attribute__((visibility("hidden"))) void set_error(const std::string &message);
}
