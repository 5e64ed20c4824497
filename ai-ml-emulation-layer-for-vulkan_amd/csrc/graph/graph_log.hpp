// Log of the graph layer, switched by the environment variable the reference uses for it: VMEL_GRAPH_SEVERITY =
// Error | Warning | Info | Debug (case-insensitive; anything else, or unset: Error).  A message is written when its
// severity is at or below the level, as one line on standard output:
//     2026-01-31 12:00:00,123 [Graph][Info] message
// (reference: common/log.cpp:29-71 for the level parsing and line format, graph/graph_log.cpp:19 for the logger's name
// and variable).  The variable is read when the first message is considered; reload() reads it again.
#pragma once

#include <sstream>
#include <string>

namespace mlel::graphlog {

enum class Severity { Error = 0, Warning = 1, Info = 2, Debug = 3 };

bool enabled(Severity severity);
void write(Severity severity, const std::string &message);
void reload();
Severity level();

}  // namespace mlel::graphlog

// The message expression is only evaluated when the severity is enabled.
#define MLEL_GRAPH_LOG(SEV, EXPR)                                                  \
    do {                                                                           \
        if (::mlel::graphlog::enabled(::mlel::graphlog::Severity::SEV)) {          \
            std::ostringstream mlel_log_os_;                                       \
            mlel_log_os_ << EXPR;                                                  \
            ::mlel::graphlog::write(::mlel::graphlog::Severity::SEV, mlel_log_os_.str()); \
        }                                                                          \
    } while (0)
