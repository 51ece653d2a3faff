// Diagnostics of the front-end: ERROR(msg, fatal) prints and, when fatal, exits with status 1
// (the reference's failure model, include/tiramisu/debug.h:109-116).  DEBUG output is
// enabled at run time with the environment variable TIRAMISU_DEBUG=<level>.
#ifndef TIRAMISU_AMD_DEBUG_H
#define TIRAMISU_AMD_DEBUG_H
#include <cstdlib>
#include <iostream>
#include <string>

namespace tiramisu {
int debug_level();
void str_dump(const std::string &str);
void str_dump(const std::string &str, const char *str2);
void str_dump(const char *str, const char *str2);
void error(const std::string &str, bool exit_program);
}  // namespace tiramisu

#define ERROR(message, exit_program)                                                   \
    do {                                                                               \
        std::cerr << "Error in " << __FILE__ << ":" << __LINE__ << " - " << (message)   \
                  << std::endl;                                                        \
        if (exit_program) std::exit(1);                                                \
    } while (0)

#define DEBUG(LEVEL, STMT)                                   \
    do {                                                     \
        if (tiramisu::debug_level() >= (LEVEL)) { STMT; }    \
    } while (0)
#define DEBUG_NO_NEWLINE(LEVEL, STMT) DEBUG(LEVEL, STMT)
#define DEBUG_NEWLINE(LEVEL) DEBUG(LEVEL, std::cout << std::endl)
#define DEBUG_INDENT(x) do { } while (0)
#define DEBUG_FCT_NAME(LEVEL) DEBUG(LEVEL, std::cout << "[" << __FUNCTION__ << "]" << std::endl)
#endif
