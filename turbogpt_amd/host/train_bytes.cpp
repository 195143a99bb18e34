// A host program over the C ABI alone (include/tg_runtime.h, tg_model.h, tg_checkpoint.h), built with
// plain g++: the shape of the reference's trainer (trainer.cpp:39-180) for the target model.
//   - weights: N(0, 0.02) matrices, residual-writing ones scaled by 1/sqrt(2 depth), gamma 1, beta 0
//   - OneCycle over the requested number of steps (trainer.cpp:61-69)
//   - training in chunks: the next chunk is launched before the previous chunk's losses are logged, so
//     host work overlaps the GPU (trainer.cpp:139-168)
//   - checkpoint at the end, resume with --load (trainer.cpp:51-55,76-80,105-121)
//   - a top-10 sample from the trained model (sampling.cpp:10-42)
//   - --log-to DIR: TensorBoard events per chunk (training_log.cpp:55-97) and DIR/report.json with the loss
//     averaged over the last 1 % of the steps (loss_summary.cpp:5-29, report.cpp:83-131)
//   - --width16 1: the reference's own network through tg_create (depth 4/8, context 4/8)
// Prints one JSON line per chunk and a final one.
#include "tg_checkpoint.h"
#include "tg_events.h"
#include "tg_model.h"
#include "tg_runtime.h"

#include <algorithm>
#include <array>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <numeric>
#include <random>
#include <stdexcept>
#include <string>
#include <vector>

namespace {

void check(int status) {
    if (status < 0)
        throw std::runtime_error(tg_error());
}

struct Options {
    std::string data, save, load, log_to;
    long long tokens = 1 << 20;
    int chunk = 16;
    bool width16 = false;
    TgModelConfig model{};
};

Options parse(int argc, char **argv) {
    Options o;
    Config &b = o.model.base;
    b.depth = 4, b.context = 256, b.batch = 8, b.learning_rate = 6e-4f, b.beta1 = 0.9f, b.beta2 = 0.95f;
    b.weight_decay = 0.1f, b.epsilon = 1e-8f, b.clip = 1.0f, b.seed = 3407, b.inflight = 1;
    b.muon_lr = 0.02f, b.momentum = 0.95f, b.ns_steps = 5;
    o.model.d_model = 256, o.model.vocab = 256, o.model.ln_eps = 1e-5f;
    for (int i = 1; i + 1 < argc; i += 2) {
        const std::string key = argv[i], value = argv[i + 1];
        if (key == "--data") o.data = value;
        else if (key == "--save") o.save = value;
        else if (key == "--load") o.load = value;
        else if (key == "--tokens") o.tokens = std::atoll(value.c_str());
        else if (key == "--chunk") o.chunk = std::atoi(value.c_str());
        else if (key == "--depth") b.depth = std::atoi(value.c_str());
        else if (key == "--context") b.context = std::atoi(value.c_str());
        else if (key == "--batch") b.batch = std::atoi(value.c_str());
        else if (key == "--d_model") o.model.d_model = std::atoi(value.c_str());
        else if (key == "--lr") b.learning_rate = float(std::atof(value.c_str()));
        else if (key == "--seed") b.seed = std::strtoull(value.c_str(), nullptr, 10);
        else if (key == "--inflight") b.inflight = std::atoi(value.c_str());
        else if (key == "--log-to") o.log_to = value;
        else if (key == "--width16") o.width16 = std::atoi(value.c_str()) != 0;
        else throw std::runtime_error("unknown option " + key);
    }
    if (o.data.empty())
        throw std::runtime_error("usage: train_bytes --data FILE [--tokens N] [--depth L] [--context T] [--batch B] "
                                 "[--d_model D] [--chunk C] [--lr R] [--seed S] [--inflight K] [--width16 1] "
                                 "[--save PATH] [--load PATH] [--log-to DIR]");
    if (o.width16) {
        o.model.d_model = 16, o.model.heads = 4, o.model.ffn = 48, o.model.ln_eps = 1e-6f;
    } else {
        o.model.heads = o.model.d_model / 64;
        o.model.ffn = 4 * o.model.d_model;
    }
    return o;
}

std::vector<float> initial_weights(const TgModelConfig &m) {
    const TgParameterLayout layout = tg_parameter_layout(&m);
    std::vector<float> w(size_t(layout.count), 0.f);
    std::mt19937_64 random(m.base.seed);
    std::normal_distribution<float> normal(0.f, 0.02f);
    const float inner = 1.0f / std::sqrt(2.0f * float(m.base.depth));
    auto fill = [&](int64_t at, int64_t count, float scale) {
        for (int64_t i = 0; i < count; ++i)
            w[size_t(at + i)] = normal(random) * scale;
    };
    auto ones = [&](int64_t at, int64_t count) { std::fill_n(w.begin() + at, count, 1.0f); };
    const int64_t d = m.d_model, f = m.ffn;
    fill(layout.embedding, int64_t(m.vocab) * d, 1), fill(layout.positions, int64_t(m.base.context) * d, 1);
    for (int l = 0; l < m.base.depth; ++l) {
        const TgLayerParameters &p = layout.layers[l];
        ones(p.ln1_g, d), ones(p.ln2_g, d);
        fill(p.qkv, 3 * d * d, 1), fill(p.attn_out, d * d, inner), fill(p.mlp_up, f * d, 1), fill(p.mlp_down, d * f, inner);
    }
    ones(layout.lnf_g, d), fill(layout.head, int64_t(m.vocab) * d, 1);
    return w;
}

// The reference's own network: flat order model.h:12-37; unit scales, N(0, 0.02) matrices, the two residual
// projections scaled by 1/sqrt(2 depth) (tests/reference.py:27-38).
std::vector<float> initial_weights_width16(const Config &c, int64_t count) {
    std::vector<float> w(size_t(count), 0.f);
    std::mt19937_64 random(c.seed);
    std::normal_distribution<float> normal(0.f, 0.02f);
    const float inner = 1.0f / std::sqrt(2.0f * float(c.depth));
    int64_t at = 0;
    auto fill = [&](int64_t n, float scale) {
        for (int64_t i = 0; i < n; ++i)
            w[size_t(at++)] = normal(random) * scale;
    };
    auto ones = [&](int64_t n) {
        for (int64_t i = 0; i < n; ++i)
            w[size_t(at++)] = 1.0f;
    };
    fill(256 * 16, 1);
    for (int l = 0; l < c.depth; ++l)
        ones(16), fill(48 * 16, 1), fill(16 * 16, inner), ones(16), fill(48 * 16, 1), fill(48 * 16, 1), fill(16 * 48, inner);
    ones(16), fill(256 * 16, 1);
    if (at != count)
        throw std::runtime_error("width-16 layout does not match the engine's parameter count");
    return w;
}

std::string sample(Engine *engine, const TgModelConfig &m) {
    const std::string prompt = "The ";
    std::vector<uint8_t> sequence(prompt.begin(), prompt.end());
    std::mt19937 random(unsigned(m.base.seed));
    std::vector<float> logits(256);
    std::array<int, 256> tokens{};
    for (int step = 0; step < 64; ++step) {
        std::vector<uint8_t> context(size_t(m.base.context), 0);
        const size_t have = std::min(sequence.size(), context.size());
        std::copy(sequence.end() - long(have), sequence.end(), context.end() - long(have));
        check(tg_predict(engine, context.data(), logits.data()));
        std::iota(tokens.begin(), tokens.end(), 0);
        std::partial_sort(tokens.begin(), tokens.begin() + 10, tokens.end(),
                          [&](int a, int b) { return logits[size_t(a)] > logits[size_t(b)]; });
        std::array<double, 10> p{};
        for (int k = 0; k < 10; ++k)
            p[size_t(k)] = std::exp(double(logits[size_t(tokens[size_t(k)])]) - double(logits[size_t(tokens[0])]));
        std::discrete_distribution<int> choose(p.begin(), p.end());
        sequence.push_back(uint8_t(tokens[size_t(choose(random))]));
    }
    std::string text;
    for (uint8_t c : sequence)
        text += (c >= 32 && c < 127 && c != '"' && c != '\\') ? char(c) : '.';
    return text;
}

double seconds_since(std::chrono::steady_clock::time_point start) {
    return std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
}

int run(int argc, char **argv) {
    Options o = parse(argc, argv);
    const TgModelConfig &m = o.model;
    const long long tokens_per_step = 1LL * m.base.batch * m.base.context;
    const int steps = int((o.tokens + tokens_per_step - 1) / tokens_per_step);
    // TRAIN_BYTES_STOP_AFTER=n ends the run after n steps of the same schedule (an interrupted run)
    const char *stop_text = std::getenv("TRAIN_BYTES_STOP_AFTER");
    const int stop = stop_text ? std::min(steps, std::atoi(stop_text)) : steps;
    Engine *engine = o.width16 ? tg_create(&m.base) : tg_create_ex(&m);
    if (!engine)
        throw std::runtime_error(tg_error());
    const int64_t count = tg_parameter_count(engine);
    const auto process_start = std::chrono::steady_clock::now();

    std::vector<float> weights, momentum(size_t(count), 0.f), variance(size_t(count), 0.f);
    TgCheckpoint state{};
    state.model = m, state.parameter_count = count;
    OneCycle schedule{steps, 0.3, 0.04, 0.000004, 0.85, 0.95};
    // loss averaged over the last max(1, ceil(steps / 100)) steps, carried through checkpoints
    // (loss_summary.cpp:5-29)
    const int average_after = std::max(0, steps - std::max(1, (steps + 99) / 100));
    std::vector<double> final_sums(size_t(m.base.context), 0.0);
    uint64_t final_batches = 0;
    if (o.load.empty()) {
        weights = o.width16 ? initial_weights_width16(m.base, count) : initial_weights(m);
    } else {
        weights.resize(size_t(count));
        TgCheckpoint header{};
        check(tg_checkpoint_inspect(o.load.c_str(), &header));
        if (header.final_loss_positions != 0 && header.final_loss_positions != m.base.context)
            throw std::runtime_error("Checkpoint loss summary does not match the context");
        state.weights = weights.data(), state.momentum = momentum.data(), state.variance = variance.data();
        state.final_loss_positions = header.final_loss_positions, state.final_loss_sums = final_sums.data();
        check(tg_checkpoint_read(o.load.c_str(), &state));
        final_batches = state.final_loss_batches;
        if (state.scheduler.total_steps != steps)
            throw std::runtime_error("Checkpoint does not match the requested run length");
        if (state.step >= uint64_t(steps))
            throw std::runtime_error("Checkpoint already reached the requested step count");
    }
    check(tg_set_weights(engine, weights.data()));
    check(tg_set_onecycle(engine, &schedule));
    if (state.step > 0)
        check(tg_set_optimizer_state(engine, momentum.data(), variance.data(), state.step));

    std::ifstream file(o.data, std::ios::binary);
    const std::vector<uint8_t> data((std::istreambuf_iterator<char>(file)), std::istreambuf_iterator<char>());
    if (data.empty())
        throw std::runtime_error("cannot read " + o.data);
    check(tg_set_data(engine, data.data(), int64_t(data.size())));

    TgEventLog *events = nullptr;
    if (!o.log_to.empty()) {
        events = tg_events_open(o.log_to.c_str(), "train_bytes");
        if (!events)
            throw std::runtime_error(tg_error());
        char text[256];
        std::snprintf(text, sizeof(text), "```\n%s d_model=%d depth=%d context=%d batch=%d heads=%d\n```",
                      o.width16 ? "swiglu48-rmsnorm-rope" : "gelu-layernorm-softmax", m.d_model, m.base.depth, m.base.context,
                      m.base.batch, m.heads);
        check(tg_events_text(events, "description", text, 0));
        check(tg_events_scalar(events, "model_bytes", double(count) * 4, 0));
        check(tg_events_scalar(events, "data_bytes", double(data.size()), 0));
        check(tg_events_scalar(events, "train_batch_size", m.base.batch, 0));
    }
    std::vector<float> last_positions(size_t(m.base.context), 0.f);

    double train_seconds = state.train_seconds;
    auto launch_start = std::chrono::steady_clock::now();
    auto launch = [&](int from) {
        const int n = std::min(o.chunk, stop - from);
        launch_start = std::chrono::steady_clock::now();
        if (n > 0)
            check(tg_train(engine, n));
        return n;
    };
    int done = int(state.step), running = launch(done);
    std::vector<float> history;
    double last_loss = 0;
    while (running) {
        history.resize(size_t(running) * size_t(m.base.context));
        check(tg_get_training_losses(engine, history.data(), running)); // waits for the chunk
        const double chunk_seconds = seconds_since(launch_start);
        train_seconds += chunk_seconds;
        const int finished = running;
        done += finished;
        running = launch(done); // the next chunk trains while this one is logged
        const float *tail = history.data() + size_t(finished - 1) * size_t(m.base.context);
        last_loss = std::accumulate(tail, tail + m.base.context, 0.0) / m.base.context;
        std::copy(tail, tail + m.base.context, last_positions.begin());
        for (int i = 0; i < finished; ++i) {
            if (done - finished + i + 1 <= average_after)
                continue;
            for (int p = 0; p < m.base.context; ++p)
                final_sums[size_t(p)] += history[size_t(i) * size_t(m.base.context) + size_t(p)];
            ++final_batches;
        }
        if (events) { // training_log.cpp:75-97; the step axis counts tokens
            const int64_t at = int64_t(done) * tokens_per_step;
            StepRates rates{};
            check(tg_onecycle_point(&schedule, done - 1, &rates));
            double used_gb = 0;
            check(tg_memory(engine, &used_gb));
            check(tg_events_scalar(events, "loss", last_loss, at));
            check(tg_events_scalar(events, "last_loss", tail[m.base.context - 1], at));
            check(tg_events_scalar(events, "bits-per-byte", tail[m.base.context - 1] / std::log(2.0), at));
            check(tg_events_scalar(events, "lr", double(m.base.learning_rate) * rates.multiplier, at));
            check(tg_events_scalar(events, "mem", used_gb, at));
            check(tg_events_scalar(events, "tokens_per_second", double(done - int(state.step)) * double(tokens_per_step) /
                                                                       std::max(train_seconds - state.train_seconds, 1e-9), at));
        }
        std::printf("{\"step\": %d, \"loss\": %.6f, \"tokens_per_s\": %.0f}\n", done, last_loss,
                    double(finished) * double(tokens_per_step) / chunk_seconds);
    }
    if (!o.save.empty()) {
        uint64_t optimizer_step = 0;
        check(tg_get_weights(engine, weights.data()));
        check(tg_get_optimizer_state(engine, momentum.data(), variance.data(), &optimizer_step));
        state.weights = weights.data(), state.momentum = momentum.data(), state.variance = variance.data();
        state.step = optimizer_step, state.scheduler = schedule, state.train_seconds = train_seconds;
        state.final_loss_positions = m.base.context, state.final_loss_sums = final_sums.data();
        state.final_loss_batches = final_batches;
        check(tg_checkpoint_write(o.save.c_str(), &state));
    }
    const std::string text = done == steps ? sample(engine, m) : "";
    if (events) {
        double mean_staleness = 0;
        int max_staleness = 0;
        check(tg_pipeline_stats(engine, &mean_staleness, &max_staleness));
        if (!text.empty())
            check(tg_events_text(events, "sample", text.c_str(), int64_t(done) * tokens_per_step));
        check(tg_events_close(events));
        // report.cpp:83-131; the sample holds printable ASCII without quotes or backslashes
        const std::string report_path = o.log_to + "/report.json";
        std::FILE *report = std::fopen(report_path.c_str(), "w");
        if (!report)
            throw std::runtime_error("Cannot write " + report_path);
        const double log2 = std::log(2.0);
        std::vector<double> average(size_t(m.base.context), 0.0);
        for (int p = 0; p < m.base.context; ++p)
            average[size_t(p)] = final_batches ? final_sums[size_t(p)] / double(final_batches) : double(last_positions[size_t(p)]);
        std::fprintf(report, "{\"architecture\":\"%s\",\"d_model\":%d,\"depth\":%d,\"ctx\":%d,\"batch\":%d,\"inflight\":%d,"
                             "\"chunk\":%d,\"seed\":%llu,\"optimizer\":\"%s\",\"learning_rate\":%.9g,\"schedule\":\"onecycle\","
                             "\"schedule_steps\":%d,\"steps\":%d,\"requested_tokens\":%lld,\"tokens\":%lld,\"parameters\":%lld,"
                             "\"final_loss\":%.9g,\"final_bpb\":%.9g,\"position_bpb\":[",
                     o.width16 ? "swiglu48-rmsnorm-rope" : "gelu-layernorm-softmax", m.d_model, m.base.depth, m.base.context,
                     m.base.batch, m.base.inflight, o.chunk, (unsigned long long)m.base.seed, o.width16 ? "muon" : "adamw",
                     double(m.base.learning_rate), steps, done, o.tokens, 1LL * done * tokens_per_step, (long long)count,
                     average.back(), average.back() / log2);
        for (int p = 0; p < m.base.context; ++p)
            std::fprintf(report, "%s%.9g", p ? "," : "", average[size_t(p)] / log2);
        std::fprintf(report, "],\"final_loss_batches\":%llu,\"sample\":\"%s\",\"mean_staleness\":%.9g,\"max_staleness\":%d,"
                             "\"training_seconds\":%.6f,\"process_seconds\":%.6f,\"tokens_per_second\":%.9g}\n",
                     (unsigned long long)final_batches, text.c_str(), mean_staleness, max_staleness, train_seconds,
                     seconds_since(process_start),
                     double(done - int(state.step)) * double(tokens_per_step) / std::max(train_seconds - state.train_seconds, 1e-9));
        if (std::fclose(report) != 0)
            throw std::runtime_error("Cannot write " + report_path);
    }
    std::printf("{\"steps\": %d, \"final_loss\": %.9g, \"train_seconds\": %.3f, \"sample\": \"%s\"}\n", done, last_loss,
                train_seconds, text.c_str());
    tg_destroy(engine);
    return 0;
}

} // namespace

int main(int argc, char **argv) {
    try {
        return run(argc, argv);
    } catch (const std::exception &error) {
        std::fprintf(stderr, "train_bytes: %s\n", error.what());
        return 1;
    }
}
