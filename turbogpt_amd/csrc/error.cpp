// Thread-local message of the last failing C-ABI call (cuda/runtime.cu:12,30-32).
#include <string>

#define TG_EXPORT extern "C" __attribute__((visibility("default")))

thread_local std::string tg_last_error;

TG_EXPORT const char *tg_error() {
    return tg_last_error.c_str();
}
TG_EXPORT const char *tgk_error() {
    return tg_last_error.c_str();
}
