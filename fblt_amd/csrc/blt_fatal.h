/*
 * Fatal-error convention of the fBLT C API (reference: csrc/core/backend.h:
 * 13-31): no return codes; a failed requirement prints one line to stderr in
 * the form "BLT Fatal Error [file:line]: ..." and ends the process with
 * EXIT_FAILURE.  Messages take printf arguments.
 */
#ifndef FBLT_AMD_BLT_FATAL_H
#define FBLT_AMD_BLT_FATAL_H

#include <stdio.h>
#include <stdlib.h>

#define BLT_FATAL(...)                                                                                             \
    do {                                                                                                           \
        fprintf(stderr, "BLT Fatal Error [%s:%d]: ", __FILE__, __LINE__);                                          \
        fprintf(stderr, __VA_ARGS__);                                                                              \
        fputc('\n', stderr);                                                                                       \
        fflush(stderr);                                                                                            \
        exit(EXIT_FAILURE);                                                                                        \
    } while (0)

#define BLT_WARN(...)                                                                                              \
    do {                                                                                                           \
        fprintf(stderr, "BLT Warning [%s:%d]: ", __FILE__, __LINE__);                                              \
        fprintf(stderr, __VA_ARGS__);                                                                              \
        fputc('\n', stderr);                                                                                       \
    } while (0)

#define BLT_REQUIRE(cond, ...)                                                                                     \
    do {                                                                                                           \
        if (!(cond)) {                                                                                             \
            fprintf(stderr, "BLT Fatal Error [%s:%d]: Requirement '%s' failed: ", __FILE__, __LINE__, #cond);      \
            fprintf(stderr, __VA_ARGS__);                                                                          \
            fputc('\n', stderr);                                                                                   \
            fflush(stderr);                                                                                        \
            exit(EXIT_FAILURE);                                                                                    \
        }                                                                                                          \
    } while (0)

#endif /* FBLT_AMD_BLT_FATAL_H */
