#include "Logger.h"

#include <chrono>
#include <cstdlib>
#include <ctime>
#include <iomanip>
#include <iostream>
#include <sstream>

Logger::Logger(const std::string &filePath, bool log2Console_, bool log2File_)
    : log2Console(log2Console_), log2File(log2File_), debugOn(getenv("TACKER_DEBUG") != nullptr)
{
    if (log2File && !filePath.empty()) {
        logFile.open(filePath, std::ios::out | std::ios::app);
        if (!logFile.is_open()) {
            std::cerr << "Error opening log file: " << filePath << std::endl;
            log2File = false;
        }
    } else {
        log2File = false;
    }
}

Logger::~Logger()
{
    if (logFile.is_open()) logFile.close();
}

std::string Logger::getTimeStamp()
{
    const auto now = std::chrono::system_clock::now();
    const std::time_t t = std::chrono::system_clock::to_time_t(now);
    const auto ms = std::chrono::duration_cast<std::chrono::milliseconds>(now.time_since_epoch()) % 1000;
    std::tm tm_buf;
    localtime_r(&t, &tm_buf);
    std::stringstream ss;
    ss << std::put_time(&tm_buf, "%Y-%m-%d %H:%M:%S") << '.' << std::setfill('0') << std::setw(3)
       << ms.count();
    return ss.str();
}

void Logger::log(LogLevel level, const std::string &message)
{
    static const char *names[] = {"DEBUG", "INFO", "WARNING", "ERROR"};
    const std::string line = "[" + getTimeStamp() + "] [" + names[(int)level] + "] " + message;
    if (log2Console) (level == LogLevel::ERROR ? std::cerr : std::cout) << line << std::endl;
    if (log2File) logFile << line << std::endl;
}

void Logger::ERROR(const std::string &message)
{
    const bool was = log2Console;
    log2Console = true;   // an error that ends the process is always shown
    log(LogLevel::ERROR, message);
    log2Console = was;
    exit(1);
}

void Logger::DEBUG(const std::string &message)
{
    if (debugOn) log(LogLevel::DEBUG, message);
}
