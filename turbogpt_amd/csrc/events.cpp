// TensorBoard event-file writer behind include/tg_events.h: the slot of the reference's
// TensorBoardLogger (tensorboard.cpp).  Host only.
//
// File = sequence of TFRecords: u64 length, u32 masked CRC-32C of those 8 bytes, payload, u32 masked
// CRC-32C of the payload (all little endian).  Payload = tensorflow.Event in protobuf wire format, written by
// hand: wall_time (1, double), step (2, varint), file_version (3) / summary (5), source_metadata (10).
// A summary value is tag (1), tensor (8), metadata (9) {plugin_data (1) {plugin_name (1)}, display_name (2),
// data_class (4)}; a scalar tensor is {dtype (1) = DT_FLOAT, tensor_shape (2) = {}, float_val (5)}, a text
// tensor {dtype = DT_STRING (7), tensor_shape {dim {size 1}}, string_val (8)}.
#include "../../include/tg_events.h"
#include "common.h"

#include <chrono>
#include <cstdio>
#include <cstring>
#include <filesystem>
#include <string>
#include <unistd.h>
#include <vector>

namespace {

struct Crc32cTable {
    uint32_t entry[4][256];
    Crc32cTable() {
        for (uint32_t i = 0; i < 256; ++i) {
            uint32_t crc = i;
            for (int bit = 0; bit < 8; ++bit)
                crc = (crc >> 1) ^ ((crc & 1) ? 0x82f63b78u : 0u);
            entry[0][i] = crc;
        }
        for (uint32_t i = 0; i < 256; ++i)
            for (int k = 1; k < 4; ++k)
                entry[k][i] = (entry[k - 1][i] >> 8) ^ entry[0][entry[k - 1][i] & 255];
    }
};
uint32_t crc32c(const unsigned char *p, size_t n) {
    static const Crc32cTable table;
    uint32_t crc = ~0u;
    for (; n >= 4; p += 4, n -= 4) { // four bytes per step
        crc ^= uint32_t(p[0]) | uint32_t(p[1]) << 8 | uint32_t(p[2]) << 16 | uint32_t(p[3]) << 24;
        crc = table.entry[3][crc & 255] ^ table.entry[2][(crc >> 8) & 255] ^ table.entry[1][(crc >> 16) & 255] ^
              table.entry[0][crc >> 24];
    }
    for (; n; ++p, --n)
        crc = (crc >> 8) ^ table.entry[0][(crc ^ *p) & 255];
    return ~crc;
}
uint32_t masked(uint32_t crc) { // TFRecord's mask: rotate right by 15, add a constant
    return ((crc >> 15) | (crc << 17)) + 0xa282ead8u;
}

// protobuf wire format, append only
struct Wire {
    std::string bytes;
    void varint(uint64_t v) {
        for (; v >= 128; v >>= 7)
            bytes.push_back(char(uint8_t(v) | 128));
        bytes.push_back(char(v));
    }
    void tag(int field, int type) { varint(uint64_t(field) << 3 | uint64_t(type)); }
    Wire &number(int field, uint64_t v) {
        tag(field, 0), varint(v);
        return *this;
    }
    Wire &blob(int field, const std::string &v) {
        tag(field, 2), varint(v.size()), bytes += v;
        return *this;
    }
    template <class T> void fixed(int field, int type, T v) {
        tag(field, type);
        unsigned char raw[sizeof(T)];
        std::memcpy(raw, &v, sizeof(T)); // x86-64 and gfx hosts are little endian
        bytes.append(reinterpret_cast<const char *>(raw), sizeof(T));
    }
    Wire &real32(int field, float v) {
        fixed(field, 5, v);
        return *this;
    }
    Wire &real64(int field, double v) {
        fixed(field, 1, v);
        return *this;
    }
};

double now_seconds() {
    return std::chrono::duration<double>(std::chrono::system_clock::now().time_since_epoch()).count();
}
std::string summary_value(const std::string &tag, const std::string &tensor, const char *plugin, int data_class) {
    Wire plugin_data, metadata, value;
    plugin_data.blob(1, plugin);
    metadata.blob(1, plugin_data.bytes).blob(2, tag).number(4, uint64_t(data_class));
    value.blob(1, tag).blob(8, tensor).blob(9, metadata.bytes);
    Wire summary;
    summary.blob(1, value.bytes);
    return summary.bytes;
}

} // namespace

struct TgEventLog {
    std::FILE *file = nullptr;
    std::string path, pending;
    static constexpr size_t BUFFER = size_t(1) << 20;

    void record(const std::string &payload) {
        unsigned char head[12];
        const uint64_t length = payload.size();
        for (int i = 0; i < 8; ++i)
            head[i] = uint8_t(length >> (8 * i));
        const uint32_t head_crc = masked(crc32c(head, 8));
        const uint32_t body_crc = masked(crc32c(reinterpret_cast<const unsigned char *>(payload.data()), payload.size()));
        for (int i = 0; i < 4; ++i)
            head[8 + i] = uint8_t(head_crc >> (8 * i));
        pending.append(reinterpret_cast<const char *>(head), 12);
        pending += payload;
        for (int i = 0; i < 4; ++i)
            pending.push_back(char(uint8_t(body_crc >> (8 * i))));
        if (pending.size() >= BUFFER)
            drain();
    }
    void drain() {
        if (!pending.empty() && std::fwrite(pending.data(), 1, pending.size(), file) != pending.size())
            throw std::runtime_error("Cannot write TensorBoard events to " + path);
        pending.clear();
    }
    void event(const std::string &summary, int64_t step) {
        Wire e;
        e.real64(1, now_seconds()).number(2, uint64_t(step)).blob(5, summary);
        record(e.bytes);
    }
};

TG_API uint32_t tg_crc32c(const void *data, size_t size) {
    return crc32c(static_cast<const unsigned char *>(data), size);
}

TG_API TgEventLog *tg_events_open(const char *directory, const char *source) {
    TgEventLog *log = nullptr;
    try {
        if (!directory || !*directory)
            throw std::runtime_error("Missing event directory");
        std::filesystem::create_directories(directory);
        char host[256] = "localhost";
        if (gethostname(host, sizeof(host) - 1) != 0 || !host[0])
            std::strcpy(host, "localhost");
        const long long seconds = (long long)(now_seconds());
        log = new TgEventLog;
        log->path = (std::filesystem::path(directory) /
                     ("events.out.tfevents." + std::to_string(seconds) + "." + host + "." + std::to_string(getpid()) + ".0"))
                        .string();
        log->file = std::fopen(log->path.c_str(), "wb");
        if (!log->file)
            throw std::runtime_error("Cannot create TensorBoard event file " + log->path);
        Wire writer, first;
        writer.blob(1, source && *source ? source : "turbogpt-mi355x");
        first.real64(1, now_seconds()).blob(3, "brain.Event:2").blob(10, writer.bytes);
        log->record(first.bytes);
        return log;
    } catch (const std::exception &error) {
        tg_last_error = error.what();
        if (log && log->file)
            std::fclose(log->file);
        delete log;
        return nullptr;
    }
}

TG_API const char *tg_events_path(TgEventLog *log) {
    return log ? log->path.c_str() : "";
}

TG_API int tg_events_scalar(TgEventLog *log, const char *tag, double value, int64_t step) {
    return guarded([&] {
        if (!log || !tag)
            throw std::runtime_error("Missing event log or tag");
        Wire tensor;
        tensor.number(1, 1).blob(2, "").real32(5, float(value)); // DT_FLOAT, rank 0
        log->event(summary_value(tag, tensor.bytes, "scalars", 1), step);
    });
}

TG_API int tg_events_text(TgEventLog *log, const char *tag, const char *text, int64_t step) {
    return guarded([&] {
        if (!log || !tag || !text)
            throw std::runtime_error("Missing event log, tag or text");
        Wire dimension, shape, tensor;
        dimension.number(1, 1);
        shape.blob(2, dimension.bytes);
        tensor.number(1, 7).blob(2, shape.bytes).blob(8, text); // DT_STRING, shape [1]
        log->event(summary_value(std::string(tag) + "/text_summary", tensor.bytes, "text", 2), step);
    });
}

TG_API int tg_events_flush(TgEventLog *log) {
    return guarded([&] {
        if (!log)
            throw std::runtime_error("Missing event log");
        log->drain();
        if (std::fflush(log->file) != 0)
            throw std::runtime_error("Cannot flush TensorBoard event file " + log->path);
    });
}

TG_API int tg_events_close(TgEventLog *log) {
    if (!log)
        return 0;
    const int status = tg_events_flush(log);
    const int closed = std::fclose(log->file);
    delete log;
    if (status == 0 && closed != 0) {
        tg_last_error = "Cannot close TensorBoard event file";
        return -1;
    }
    return status;
}
