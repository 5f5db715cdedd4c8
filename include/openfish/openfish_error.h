/*
 * Log level and logging macros of the openfish API (reference
 * include/openfish/openfish_error.h:44-106, src/error.c:33-41).  The level is
 * one process-wide value, OPENFISH_LOG_VERB by default; messages go to stderr.
 */
#ifndef OPENFISH_ERROR_H
#define OPENFISH_ERROR_H

#include <stdio.h>
#include <string.h>

#ifdef __cplusplus
extern "C" {
#endif

enum openfish_log_level_opt {
    OPENFISH_LOG_OFF,  /* nothing */
    OPENFISH_LOG_ERR,  /* errors */
    OPENFISH_LOG_WARN, /* + warnings */
    OPENFISH_LOG_INFO, /* + information */
    OPENFISH_LOG_VERB, /* + verbose */
    OPENFISH_LOG_DBUG, /* + debugging */
    OPENFISH_LOG_TRAC  /* + tracing */
};

enum openfish_log_level_opt get_openfish_log_level(void);
void set_openfish_log_level(enum openfish_log_level_opt level);

#define openfish_log_level get_openfish_log_level()

/* one formatter behind every macro; `where` adds the " At file:line" suffix */
void openfish_log_emit(enum openfish_log_level_opt need, const char *tag, const char *colour,
                       const char *func, const char *file, int line, int where, const char *fmt, ...)
#if defined(__GNUC__)
    __attribute__((format(printf, 8, 9)))
#endif
    ;

#define OPENFISH_LOG_TRACE(msg, ...) \
    openfish_log_emit(OPENFISH_LOG_TRAC, "OPENFISH_DEBUG", NULL, __func__, __FILE__, __LINE__, 1, msg, __VA_ARGS__)
#define OPENFISH_LOG_DEBUG(msg, ...) \
    openfish_log_emit(OPENFISH_LOG_DBUG, "OPENFISH_DEBUG", NULL, __func__, __FILE__, __LINE__, 1, msg, __VA_ARGS__)
#define OPENFISH_VERBOSE(msg, ...) \
    openfish_log_emit(OPENFISH_LOG_VERB, "OPENFISH_INFO", NULL, __func__, __FILE__, __LINE__, 0, msg, __VA_ARGS__)
#define OPENFISH_INFO(msg, ...) \
    openfish_log_emit(OPENFISH_LOG_INFO, "OPENFISH_INFO", "\033[1;34m", __func__, __FILE__, __LINE__, 0, msg, __VA_ARGS__)
#define OPENFISH_WARNING(msg, ...) \
    openfish_log_emit(OPENFISH_LOG_WARN, "OPENFISH_WARNING", "\033[1;33m", __func__, __FILE__, __LINE__, 1, msg, __VA_ARGS__)
#define OPENFISH_ERROR(msg, ...) \
    openfish_log_emit(OPENFISH_LOG_ERR, "OPENFISH_ERROR", "\033[1;31m", __func__, __FILE__, __LINE__, 1, msg, __VA_ARGS__)

#ifdef __cplusplus
}
#endif

#endif /* OPENFISH_ERROR_H */
