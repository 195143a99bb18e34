// A host program over the C ABI alone (include/tg_runtime.h, tg_model.h, tg_checkpoint.h), built with
// plain g++: the shape of the reference's trainer (trainer.cpp:39-180) for the target model.
//   - weights: N(0, 0.02) matrices, residual-writing ones scaled by 1/sqrt(2 depth), gamma 1, beta 0
//   - OneCycle over the requested number of steps (trainer.cpp:61-69)
//   - training in chunks: the next chunk is launched before the previous chunk's losses are logged, so
//     host work overlaps the GPU (trainer.cpp:139-168)
//   - checkpoint at the end, resume with --load (trainer.cpp:51-55,76-80,105-121)
//   - a top-10 sample from the trained model (sampling.cpp:10-42)
//   - --log-to DIR: TensorBoard events per chunk (training_log.cpp:55-97) and DIR/report.json with the loss
//     averaged over the last 1 % of the steps (loss_summary.cpp:5-29, report.cpp:82-131)
//   - --width16 1: the reference's own network through tg_create (depth 4/8, context 4/8)
// Standard output carries the reference's JSON lines, key for key and in its order: {"config":{...}} once
// (report.cpp:46-59), one {"step":...} object per chunk (report.cpp:61-80) and {"summary":{...}} at the end
// (report.cpp:82-117); keys the reference does not have (d_model, heads, ffn, vocab, loss, steps, parameters,
// final_loss_batches, last_loss) follow the reference's inside each object.
#include "tg_checkpoint.h"
#include "tg_events.h"
#include "tg_model.h"
#include "tg_runtime.h"

#include <limits>
#include <algorithm>
#include <array>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iomanip>
#include <iostream>
#include <sstream>
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

// The ten likeliest next bytes, likeliest first, with their logits: one pass with a small sorted list.
struct Candidate {
    int byte;
    float logit;
};
std::array<Candidate, 10> likeliest(const std::vector<float> &logits) {
    std::array<Candidate, 10> best;
    best.fill({0, -std::numeric_limits<float>::infinity()});
    for (int byte = 0; byte < 256; ++byte) {
        const float logit = logits[size_t(byte)];
        if (!(logit > best.back().logit))
            continue;
        size_t place = best.size() - 1;
        for (; place > 0 && logit > best[place - 1].logit; --place)
            best[place] = best[place - 1];
        best[place] = {byte, logit};
    }
    return best;
}

// Text continued byte by byte from the trained model through tg_predict (the slot of sampling.cpp:10-42): the window
// holds the last `context` bytes, right-aligned behind zeros; each byte is drawn from the softmax over the ten
// likeliest, by inverting the cumulative weights at a uniform number from a generator seeded with the model's seed.
std::string sample(Engine *engine, const TgModelConfig &m) {
    const int generated = 64;
    std::vector<uint8_t> window(size_t(m.base.context), 0);
    std::string text = "The ";
    auto push = [&](uint8_t byte) {
        std::move(window.begin() + 1, window.end(), window.begin());
        window.back() = byte;
    };
    for (char c : text)
        push(uint8_t(c));
    uint64_t state = uint64_t(m.base.seed) * 0x9e3779b97f4a7c15ull + 1;
    auto uniform = [&]() { // xorshift64*: 53 random bits as a number in [0, 1)
        state ^= state >> 12, state ^= state << 25, state ^= state >> 27;
        return double((state * 0x2545f4914f6cdd1dull) >> 11) * (1.0 / 9007199254740992.0);
    };
    std::vector<float> logits(256);
    for (int n = 0; n < generated; ++n) {
        check(tg_predict(engine, window.data(), logits.data()));
        const auto best = likeliest(logits);
        double weight[10], total = 0;
        for (size_t k = 0; k < best.size(); ++k)
            total += weight[k] = std::exp(double(best[k].logit) - double(best[0].logit));
        double left = uniform() * total;
        size_t pick = 0;
        while (pick + 1 < best.size() && left >= weight[pick])
            left -= weight[pick++];
        const uint8_t byte = uint8_t(best[pick].byte);
        push(byte);
        text += (byte >= 32 && byte < 127 && byte != '"' && byte != '\\') ? char(byte) : '.';
    }
    return text;
}

double seconds_since(std::chrono::steady_clock::time_point start) {
    return std::chrono::duration<double>(std::chrono::steady_clock::now() - start).count();
}

// a JSON string literal: control characters and bytes beyond ASCII as \u00XX (report.cpp:9-43)
void json_string(std::ostream &out, const std::string &value) {
    static const char hex[] = "0123456789abcdef";
    out << '"';
    for (unsigned char byte : value) {
        if (byte == '"' || byte == '\\')
            out << '\\' << char(byte);
        else if (byte == '\n')
            out << "\\n";
        else if (byte == '\r')
            out << "\\r";
        else if (byte == '\t')
            out << "\\t";
        else if (byte < 0x20 || byte >= 0x80)
            out << "\\u00" << hex[byte >> 4] << hex[byte & 15];
        else
            out << char(byte);
    }
    out << '"';
}
const char *architecture(const Options &o) { return o.width16 ? "swiglu48-rmsnorm-rope" : "gelu-layernorm-softmax"; }
const char *optimizer(const Options &o) { return o.width16 ? "muon" : "adamw"; }

// {"config":{...}}: the keys of report.cpp:46-59 in its order, then the model shape the reference has no field for
void log_config(Engine *engine, const Options &o, const OneCycle &schedule, int steps, int64_t dataset_bytes) {
    const TgModelConfig &m = o.model;
    std::cout << "{\"config\":{\"architecture\":\"" << architecture(o) << "\",\"depth\":" << m.base.depth
              << ",\"ctx\":" << m.base.context << ",\"batch\":" << m.base.batch << ",\"inflight\":" << m.base.inflight
              << ",\"chunk\":" << o.chunk << ",\"optimizer\":\"" << optimizer(o)
              << "\",\"parameters\":" << tg_parameter_count(engine) << ",\"blocks\":" << tg_blocks(engine)
              << ",\"shared_bytes\":" << tg_shared_bytes(engine) << ",\"steps\":" << steps
              << ",\"dataset_bytes\":" << dataset_bytes << ",\"schedule\":\"onecycle\""
              << ",\"warmup_fraction\":" << schedule.warmup_fraction
              << ",\"initial_lr_fraction\":" << schedule.initial_lr_fraction
              << ",\"final_lr_fraction\":" << schedule.final_lr_fraction << ",\"low_momentum\":" << schedule.low_momentum
              << ",\"high_momentum\":" << schedule.high_momentum << ",\"d_model\":" << m.d_model
              << ",\"heads\":" << m.heads << ",\"ffn\":" << m.ffn << ",\"vocab\":" << m.vocab << "}}" << std::endl;
}

// one object per chunk: report.cpp:61-80 (losses of the chunk's last step, cumulative time and rate), then "loss"
void log_step(const Options &o, const OneCycle &schedule, const float *losses, int done, double train_seconds) {
    const TgModelConfig &m = o.model;
    const int64_t per_step = int64_t(m.base.batch) * m.base.context;
    const double log2 = std::log(2.0);
    std::cout << "{\"step\":" << done << ",\"tokens\":" << done * per_step
              << ",\"last_bpb\":" << losses[m.base.context - 1] / log2 << ",\"position_bpb\":[";
    for (int position = 0; position < m.base.context; ++position)
        std::cout << (position ? "," : "") << losses[position] / log2;
    StepRates rates{};
    check(tg_onecycle_point(&schedule, done - 1, &rates));
    std::cout << "],\"adam_lr\":" << m.base.learning_rate * rates.multiplier
              << ",\"muon_lr\":" << m.base.muon_lr * rates.multiplier << ",\"momentum\":" << rates.momentum
              << ",\"train_seconds\":" << train_seconds << ",\"tokens_per_second\":" << done * per_step / train_seconds
              << ",\"loss\":" << std::accumulate(losses, losses + m.base.context, 0.0) / m.base.context << "}" << std::endl;
}

struct RunReport {
    int steps, done;
    std::vector<double> final_losses; // per position, averaged over the last 1 % of the steps
    uint64_t final_loss_batches;
    std::string sample;
    double initialize_seconds, load_seconds, train_seconds, sample_seconds, total, mean_staleness, last_loss;
    int max_staleness;
    int64_t parameters;
};
// the summary object: report.cpp:82-117 key for key, then the added keys
void report(std::ostream &out, const Options &o, const OneCycle &schedule, const RunReport &r) {
    const TgModelConfig &m = o.model;
    const double log2 = std::log(2.0), final_loss = r.final_losses.back();
    const int64_t tokens = r.steps * (int64_t(m.base.batch) * m.base.context);
    out << std::setprecision(10) << "{\"architecture\":\"" << architecture(o) << "\",\"depth\":" << m.base.depth
        << ",\"ctx\":" << m.base.context << ",\"batch\":" << m.base.batch << ",\"inflight\":" << m.base.inflight
        << ",\"chunk\":" << o.chunk << ",\"seed\":" << m.base.seed << ",\"optimizer\":\"" << optimizer(o)
        << "\",\"learning_rate\":" << m.base.learning_rate << ",\"muon_lr\":" << m.base.muon_lr
        << ",\"schedule\":\"onecycle\",\"schedule_steps\":" << r.steps
        << ",\"warmup_fraction\":" << schedule.warmup_fraction << ",\"initial_lr_fraction\":" << schedule.initial_lr_fraction
        << ",\"final_lr_fraction\":" << schedule.final_lr_fraction << ",\"low_momentum\":" << schedule.low_momentum
        << ",\"high_momentum\":" << schedule.high_momentum << ",\"requested_tokens\":" << o.tokens << ",\"tokens\":" << tokens
        << ",\"final_loss\":" << final_loss << ",\"final_bpb\":" << final_loss / log2 << ",\"position_bpb\":[";
    for (size_t position = 0; position < r.final_losses.size(); ++position)
        out << (position ? "," : "") << r.final_losses[position] / log2;
    out << "],\"sample\":";
    json_string(out, r.sample);
    out << ",\"initialization_seconds\":" << r.initialize_seconds << ",\"mean_staleness\":" << r.mean_staleness
        << ",\"max_staleness\":" << r.max_staleness << ",\"dataset_load_seconds\":" << r.load_seconds
        << ",\"training_seconds\":" << r.train_seconds << ",\"sample_seconds\":" << r.sample_seconds
        << ",\"process_seconds\":" << r.total << ",\"tokens_per_second\":" << tokens / r.train_seconds
        << ",\"sample_temperature\":1.0,\"d_model\":" << m.d_model << ",\"steps\":" << r.done
        << ",\"parameters\":" << r.parameters << ",\"final_loss_batches\":" << r.final_loss_batches
        << ",\"last_loss\":" << r.last_loss << "}";
}

int run(int argc, char **argv) {
    Options o = parse(argc, argv);
    const TgModelConfig &m = o.model;
    const long long tokens_per_step = 1LL * m.base.batch * m.base.context;
    const int steps = int((o.tokens + tokens_per_step - 1) / tokens_per_step);
    // TRAIN_BYTES_STOP_AFTER=n ends the run after n steps of the same schedule (an interrupted run)
    const char *stop_text = std::getenv("TRAIN_BYTES_STOP_AFTER");
    const int stop = stop_text ? std::min(steps, std::atoi(stop_text)) : steps;
    const auto process_start = std::chrono::steady_clock::now();
    std::cout << std::setprecision(9);
    Engine *engine = o.width16 ? tg_create(&m.base) : tg_create_ex(&m);
    if (!engine)
        throw std::runtime_error(tg_error());
    const int64_t count = tg_parameter_count(engine);

    std::vector<float> weights, momentum(size_t(count), 0.f), variance(size_t(count), 0.f);
    TgCheckpoint state{};
    state.model = m, state.parameter_count = count;
    OneCycle schedule{steps, 0.3, 0.04, 0.000004, 0.85, 0.95};
    // loss averaged over the last max(1, ceil(steps / 100)) steps, carried through checkpoints
    // (loss_summary.cpp:5-29)
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
    const double initialize_seconds = seconds_since(process_start);
    // what a resumed run starts from: its rate counts only its own steps and seconds
    const int start_step = int(state.step);
    const double start_seconds = state.train_seconds;

    const auto load_start = std::chrono::steady_clock::now();
    std::ifstream file(o.data, std::ios::binary);
    const std::vector<uint8_t> data((std::istreambuf_iterator<char>(file)), std::istreambuf_iterator<char>());
    if (data.empty())
        throw std::runtime_error("cannot read " + o.data);
    check(tg_set_data(engine, data.data(), int64_t(data.size())));
    const double load_seconds = seconds_since(load_start);
    log_config(engine, o, schedule, steps, int64_t(data.size()));

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
        for (int i = 0; i < finished; ++i)
            check(tg_final_loss_add(steps, m.base.context, done - finished + i + 1,
                                    history.data() + size_t(i) * size_t(m.base.context), final_sums.data(), &final_batches));
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
            check(tg_events_scalar(events, "tokens_per_second", double(done - start_step) * double(tokens_per_step) /
                                                                       std::max(train_seconds - start_seconds, 1e-9), at));
        }
        (void)chunk_seconds;
        log_step(o, schedule, tail, done, train_seconds);
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
    const auto sample_start = std::chrono::steady_clock::now();
    const std::string text = done == steps ? sample(engine, m) : "";
    const double sample_seconds = seconds_since(sample_start);
    RunReport r{};
    r.steps = steps, r.done = done, r.final_loss_batches = final_batches, r.sample = text;
    r.final_losses.resize(size_t(m.base.context));
    for (int p = 0; p < m.base.context; ++p)
        r.final_losses[size_t(p)] = final_batches ? final_sums[size_t(p)] / double(final_batches) : double(last_positions[size_t(p)]);
    r.initialize_seconds = initialize_seconds, r.load_seconds = load_seconds, r.train_seconds = train_seconds;
    r.sample_seconds = sample_seconds, r.last_loss = last_loss, r.parameters = count;
    check(tg_pipeline_stats(engine, &r.mean_staleness, &r.max_staleness));
    if (events) {
        if (!text.empty())
            check(tg_events_text(events, "sample", text.c_str(), int64_t(done) * tokens_per_step));
        check(tg_events_close(events));
    }
    r.total = seconds_since(process_start);
    std::cout << "{\"summary\":";
    report(std::cout, o, schedule, r);
    std::cout << "}" << std::endl;
    if (events) { // DIR/report.json holds the summary object (report.cpp:119-131)
        const std::string report_path = o.log_to + "/report.json";
        std::ofstream out(report_path);
        report(out, o, schedule, r);
        out << '\n';
        if (!out)
            throw std::runtime_error("Cannot write " + report_path);
    }
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
