// Logging set-up of the host core (include/armnn/Utils.hpp:13-28).
#pragma once

namespace armnn
{
enum class LogSeverity
{
    Trace,
    Debug,
    Info,
    Warning,
    Error,
    Fatal
};

/// Messages of `severity` and above go to standard output when printToStandardOutput is set; until this is called the core
/// prints warnings and errors to standard error.  printToDebugOutput is accepted and ignored (it names a Windows facility).
void ConfigureLogging(bool printToStandardOutput, bool printToDebugOutput, LogSeverity severity);

/// what ConfigureLogging last set: used by the core's own messages
bool LogsAt(LogSeverity severity);
bool LogsToStandardOutput();
} // namespace armnn
