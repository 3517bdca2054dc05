// error.h -- per-thread last-error text behind coral_last_error().
#pragma once
namespace coral {
// records a printf-style message for the calling thread and returns `code`
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
}
