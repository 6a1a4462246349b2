// Logger.h -- timestamped console / file log (src/Logger.h of the reference).
// ERROR logs and exits with status 1 (:38-41); DEBUG is printed only when the
// environment variable TACKER_DEBUG is set (the reference gates it on the CMake
// build type, :43-49).
#pragma once
#include <fstream>
#include <string>

enum class LogLevel { DEBUG, INFO, WARNING, ERROR };

class Logger {
public:
    Logger(const std::string &filePath, bool log2Console = true, bool log2File = false);
    ~Logger();
    void log(LogLevel level, const std::string &message);
    void INFO(const std::string &message) { log(LogLevel::INFO, message); }
    void WARNING(const std::string &message) { log(LogLevel::WARNING, message); }
    [[noreturn]] void ERROR(const std::string &message);
    void DEBUG(const std::string &message);
    void setConsole(bool on) { log2Console = on; }

private:
    std::ofstream logFile;
    bool log2Console;
    bool log2File;
    bool debugOn;
    std::string getTimeStamp();
};
