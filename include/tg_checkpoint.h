/*
 * Training checkpoints in PyTorch's zip container (readable with torch.load(path, weights_only=True)).
 * Host-only functions: no GPU call is made.  They take the slot of save_training_state /
 * load_training_state (checkpoint.h:7-17, checkpoint.cpp:506-579) for the target model: the file holds
 * the same nested dictionary
 *     model        : depth, context, weights            (+ d_model, heads, vocab, ffn for the target model)
 *     opt          : momentum, variance, step
 *     lr_scheduler : total_steps, step, warmup_fraction, initial_lr_fraction, final_lr_fraction,
 *                    low_momentum, high_momentum
 *     trainer      : train_seconds, final_loss_sums, final_loss_batches
 * with the reference's storage numbering (archive/data/0 .. 14, checkpoint.cpp:155-197) and its container
 * records (.format_version, .storage_alignment, byteorder, version, .data/serialization_id); the width
 * fields are storages 15 .. 18.  A width-16 file written here loads through the reference's
 * load_training_state, and a file the reference wrote (storages 0 .. 14 only) reads here as the width-16
 * network.  Records are stored uncompressed, 64-byte aligned, with CRC-32.  Sizes and offsets are the
 * 32-bit ZIP fields the reference's reader uses: a file holds less than 4 GiB (about 357 M parameters);
 * tg_checkpoint_write refuses a larger state before it writes anything.
 * Same status convention as tg_runtime.h: 0 on success, -1 with the reason in tg_error().
 */
#ifndef TG_CHECKPOINT_H
#define TG_CHECKPOINT_H
#include "tg_runtime.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct TgCheckpoint {
    TgModelConfig model;         /* only depth, context, d_model, heads, vocab, ffn are stored */
    int64_t parameter_count;     /* elements of each of weights / momentum / variance */
    float *weights, *momentum, *variance;
    uint64_t step;
    OneCycle scheduler;          /* total_steps == 0: no schedule */
    double train_seconds;
    int64_t final_loss_positions; /* elements of final_loss_sums (0 or context) */
    double *final_loss_sums;
    uint64_t final_loss_batches;
} TgCheckpoint;

/* Writes `path` atomically (temporary file in the same directory, then rename), as
 * checkpoint.cpp:20-31,554-579 does. */
TG_API int tg_checkpoint_write(const char *path, const TgCheckpoint *checkpoint);
/* Fills every scalar field, `model` and the two counts; leaves the four pointers untouched. */
TG_API int tg_checkpoint_inspect(const char *path, TgCheckpoint *header);
/* Reads the arrays into the caller's buffers, whose sizes (parameter_count, final_loss_positions)
 * must equal the file's; verifies every record's CRC-32 and the container metadata, and rejects
 * a file whose architecture fields differ from `checkpoint->model` when d_model there is non-zero
 * (checkpoint.cpp:524-551: "Checkpoint architecture mismatch"). */
TG_API int tg_checkpoint_read(const char *path, TgCheckpoint *checkpoint);

/* The loss summary that travels through checkpoints (FinalLossAverage::add, loss_summary.cpp:5-29): adds the
 * per-position losses of step `completed_step` (1-based) to sums[positions] and counts it in *batches when the
 * step lies in the last max(1, ceil(total_steps / 100)) steps of the run; earlier steps change nothing. */
TG_API int tg_final_loss_add(int total_steps, int positions, int completed_step, const float *losses, double *sums,
                             uint64_t *batches);

#ifdef __cplusplus
}
#endif
#endif
