// The calling thread's last error text, shared by the host translation units of the library.
#pragma once

namespace hstu {

// formats the text that hstu_last_error() returns on this thread and hands `code` back
int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

}  // namespace hstu
