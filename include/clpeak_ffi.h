/* clpeak's embedding C ABI, served by the MI355X backend.
 *
 * These are the six entry points of the reference's GUI bridge (src/ffi/clpeak_ffi.h:26-104), with
 * the same names, argument meaning, ownership rules and return codes, so that a front end written
 * against the reference's library loads libclpeak_host.so instead and runs an MI355X unchanged.
 * The only backend compiled in is "ROCm".
 *
 * String ownership: `char *` results are malloc'd UTF-8; release them with clpeak_free_string().
 * `const char *` results are static.  An event string handed to the callback belongs to the
 * callee, which releases it with clpeak_free_string() once consumed (src/ffi/clpeak_ffi.h:40-45).
 */
#ifndef CLPEAK_FFI_H
#define CLPEAK_FFI_H

#define CLPEAK_FFI_EXPORT __attribute__((visibility("default")))

#ifdef __cplusplus
extern "C" {
#endif

/* src/ffi/clpeak_ffi.h:28 -- version string, static. */
CLPEAK_FFI_EXPORT const char *clpeak_version(void);

/* src/ffi/clpeak_ffi.h:30-34 -- device catalog as the inventory document
 *   {"backends":[{"name","available","platforms":[{"index","name","devices":[{"index","name","type",
 *     "driver","computeUnits","clockMHz","globalMemBytes","fp16","fp64"}]}]}]}
 * (serializer: src/common/inventory.cpp:11-73; zero / empty fields are omitted). */
CLPEAK_FFI_EXPORT char *clpeak_copy_backend_catalog_json(void);

/* src/ffi/clpeak_ffi.h:36 */
CLPEAK_FFI_EXPORT void clpeak_free_string(char *s);

/* src/ffi/clpeak_ffi.h:46-66 -- one JSON document per run event, field "t" names the kind:
 * backend_begin, device, test_begin, metric, test_skipped, test_end, device_end, backend_end, note,
 * done {status, cancelled}.  `done` is always the last event of a launch.  Numbers are written in
 * the classic locale with 4 decimals (src/ffi/logger_ffi.cpp:36-50).  Callbacks fire on the thread
 * that called clpeak_launch(). */
typedef void (*ClpeakEventCallback)(void *user_data, char *event_json);

#define CLPEAK_RUN_OK         0    /* all backends completed                        */
/* > 0: OR'd backend error statuses                                                  */
#define CLPEAK_RUN_BAD_ARGS  (-1)  /* argv rejected; nothing ran                    */
#define CLPEAK_RUN_CANCELLED (-2)  /* clpeak_request_cancel() honoured              */
#define CLPEAK_RUN_BUSY      (-3)  /* another launch is in progress; no done event  */

/* src/ffi/clpeak_ffi.h:68-82, src/ffi/clpeak_ffi.cpp:161-225 -- blocking run.  argv follows the CLI
 * flag grammar (argv[0] is skipped like a program name); --help / --version are rejected;
 * --xml-file / --json-file / --csv-file are honoured at the end of the run, also after a
 * cancellation.  Never exits the process. */
CLPEAK_FFI_EXPORT int clpeak_launch(int argc, const char **argv, ClpeakEventCallback on_event, void *user_data);

/* src/ffi/clpeak_ffi.h:84-90 -- cooperative cancel, observed at test boundaries; any thread; the
 * flag resets at the start of the next launch. */
CLPEAK_FFI_EXPORT void clpeak_request_cancel(void);

/* src/ffi/clpeak_ffi.h:92-104 -- load a saved XML / JSON / CSV result file (format_version 2) and
 * return it as the JSON dump document; NULL when unreadable, rejected or empty. */
CLPEAK_FFI_EXPORT char *clpeak_load_result_file_json(const char *path);

#ifdef __cplusplus
}
#endif
#endif /* CLPEAK_FFI_H */
