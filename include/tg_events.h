/*
 * TensorBoard event files (TFRecord framing with masked CRC-32C around protobuf-encoded Event messages).
 * Host-only functions: no GPU call is made.  They take the slot of the reference's TensorBoardLogger
 * (tensorboard.h:10-30, tensorboard.cpp:178-254): scalars and text are written as tensor summaries with
 * the "scalars" / "text" plugin metadata, the first record is the file-version event "brain.Event:2".
 * Records are buffered and reach the file when the buffer fills, on tg_events_flush and on tg_events_close.
 * Same status convention as tg_runtime.h: 0 on success, -1 (NULL for tg_events_open) with the reason in
 * tg_error().
 */
#ifndef TG_EVENTS_H
#define TG_EVENTS_H
#include "tg_runtime.h"
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct TgEventLog TgEventLog;

/* Creates `directory` if needed and in it events.out.tfevents.<seconds>.<host>.<pid>.0
 * (tensorboard.cpp:178-196); `source` names the writer in the file-version event. */
TG_API TgEventLog *tg_events_open(const char *directory, const char *source);
TG_API const char *tg_events_path(TgEventLog *log);
/* One scalar point: tag, float32 value, step (tensorboard.cpp:221-239). */
TG_API int tg_events_scalar(TgEventLog *log, const char *tag, double value, int64_t step);
/* One text point under "<tag>/text_summary" (tensorboard.cpp:241-246). */
TG_API int tg_events_text(TgEventLog *log, const char *tag, const char *text, int64_t step);
TG_API int tg_events_flush(TgEventLog *log);
/* Flushes and frees; the status reports a failed final write. */
TG_API int tg_events_close(TgEventLog *log);
/* CRC-32C (Castagnoli, reflected polynomial 0x82f63b78) as the framing uses it (tensorboard.cpp:72-105). */
TG_API uint32_t tg_crc32c(const void *data, size_t size);

#ifdef __cplusplus
}
#endif
#endif
