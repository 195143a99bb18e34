// Test infrastructure only.  C linkage around three host-only translation units of the reference, compiled
// from the reference tree where they lie (oracle/Makefile, target ref): the checkpoint writer / reader
// (checkpoint.cpp:506-579), the loss summary that travels through checkpoints (loss_summary.cpp:5-29) and the
// TensorBoard event writer (tensorboard.cpp:178-254).  Nothing of theirs is copied here; the tests use these
// entry points to cross-read files between the reference's code and the library's.
#include "checkpoint.h"
#include "loss_summary.h"
#include "tensorboard.h"

#include <cstdint>
#include <cstring>
#include <string>

namespace {
thread_local std::string last_error;
template <class F> int guarded(F &&body) {
    try {
        body();
        return 0;
    } catch (const std::exception &error) {
        last_error = error.what();
        return -1;
    }
}
Config config_of(int depth, int context) {
    Config config{};
    config.depth = depth, config.context = context;
    return config;
}
} // namespace

extern "C" const char *tgref_io_error() { return last_error.c_str(); }

// scalars: [step, total_steps, final_loss_batches] ; reals: [warmup, initial, final, low, high, train_seconds]
extern "C" int tgref_checkpoint_save(const char *path, int depth, int context, int64_t count, const float *weights,
                                     const float *momentum, const float *variance, const int64_t *scalars,
                                     const double *reals, const double *loss_sums) {
    return guarded([&] {
        TrainingState state;
        state.weights.assign(weights, weights + count);
        state.momentum.assign(momentum, momentum + count);
        state.variance.assign(variance, variance + count);
        state.step = uint64_t(scalars[0]);
        state.scheduler = OneCycle{int(scalars[1]), reals[0], reals[1], reals[2], reals[3], reals[4]};
        state.train_seconds = reals[5];
        state.final_loss_sums.assign(loss_sums, loss_sums + context);
        state.final_loss_batches = uint64_t(scalars[2]);
        save_training_state(path, config_of(depth, context), state);
    });
}

extern "C" int tgref_checkpoint_load(const char *path, int depth, int context, int64_t count, float *weights,
                                     float *momentum, float *variance, int64_t *scalars, double *reals,
                                     double *loss_sums) {
    return guarded([&] {
        const TrainingState state = load_training_state(path, config_of(depth, context));
        if (int64_t(state.weights.size()) != count || int64_t(state.final_loss_sums.size()) != context)
            throw std::runtime_error("unexpected array sizes");
        std::memcpy(weights, state.weights.data(), size_t(count) * 4);
        std::memcpy(momentum, state.momentum.data(), size_t(count) * 4);
        std::memcpy(variance, state.variance.data(), size_t(count) * 4);
        std::memcpy(loss_sums, state.final_loss_sums.data(), size_t(context) * 8);
        scalars[0] = int64_t(state.step), scalars[1] = state.scheduler.total_steps, scalars[2] = int64_t(state.final_loss_batches);
        reals[0] = state.scheduler.warmup_fraction, reals[1] = state.scheduler.initial_lr_fraction;
        reals[2] = state.scheduler.final_lr_fraction, reals[3] = state.scheduler.low_momentum;
        reals[4] = state.scheduler.high_momentum, reals[5] = state.train_seconds;
    });
}

// FinalLossAverage over `steps` consecutive steps starting at completed step `first`: sums, batches, average
extern "C" int tgref_final_loss(int total_steps, int positions, int first, int steps, const float *losses, double *sums,
                                uint64_t *batches, float *average) {
    return guarded([&] {
        FinalLossAverage summary(total_steps, positions, std::vector<double>(sums, sums + positions), *batches);
        for (int i = 0; i < steps; ++i)
            summary.add(first + i, std::vector<float>(losses + size_t(i) * positions, losses + size_t(i + 1) * positions));
        std::memcpy(sums, summary.sums().data(), size_t(positions) * 8);
        *batches = summary.batches();
        const std::vector<float> mean = summary.average();
        std::memcpy(average, mean.data(), size_t(positions) * 4);
    });
}

extern "C" void *tgref_events_open(const char *directory) {
    void *logger = nullptr;
    guarded([&] { logger = new TensorBoardLogger(directory); });
    return logger;
}
extern "C" int tgref_events_scalar(void *logger, const char *tag, double value, int64_t step) {
    return guarded([&] { static_cast<TensorBoardLogger *>(logger)->scalar(tag, value, step); });
}
extern "C" int tgref_events_text(void *logger, const char *tag, const char *text, int64_t step) {
    return guarded([&] { static_cast<TensorBoardLogger *>(logger)->text(tag, text, step); });
}
extern "C" int tgref_events_close(void *logger) {
    return guarded([&] { delete static_cast<TensorBoardLogger *>(logger); });
}
