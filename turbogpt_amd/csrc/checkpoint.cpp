// Training checkpoints in PyTorch's zip container, host only.  Takes the slot of the reference's
// save_training_state / load_training_state (checkpoint.cpp:506-579): same dictionary, same storage
// numbering, readable with torch.load(..., weights_only=True).
//
// Container facts relied on (PyTorch's serialization format 3): a ZIP archive of *stored* records under
// one directory prefix; <prefix>/data.pkl is a protocol-2 pickle in which a tensor is
// torch._utils._rebuild_tensor_v2(persistent storage id, offset, size, stride, requires_grad, hooks) and
// the persistent id is the tuple ('storage', torch.<Type>Storage, key, 'cpu', numel); the bytes of storage
// `key` are the record <prefix>/data/<key>, little endian.  Records start on 64-byte boundaries (padding
// goes into a local-header extra field).  Writing streams each array to the file; nothing the size of the
// model is held besides the caller's arrays.
#include "common.h"
#include "../../include/tg_checkpoint.h"
#include "../../include/tg_model.h"

#include <algorithm>
#include <cerrno>
#include <cstdio>
#include <cstring>
#include <map>
#include <memory>
#include <vector>

namespace {

// ---- CRC-32 (IEEE 802.3, the ZIP polynomial), 8 bytes per step ----------------------------------
struct CrcTables {
    uint32_t t[8][256];
    CrcTables() {
        for (uint32_t i = 0; i < 256; ++i) {
            uint32_t c = i;
            for (int k = 0; k < 8; ++k)
                c = (c >> 1) ^ (0xedb88320u & (0u - (c & 1u)));
            t[0][i] = c;
        }
        for (uint32_t i = 0; i < 256; ++i)
            for (int s = 1; s < 8; ++s)
                t[s][i] = (t[s - 1][i] >> 8) ^ t[0][t[s - 1][i] & 0xff];
    }
};
uint32_t crc32_of(const void *data, size_t size, uint32_t crc = 0) {
    static const CrcTables tables;
    const unsigned char *p = static_cast<const unsigned char *>(data);
    crc = ~crc;
    while (size >= 8) {
        uint32_t lo, hi;
        std::memcpy(&lo, p, 4);
        std::memcpy(&hi, p + 4, 4);
        lo ^= crc;
        crc = tables.t[7][lo & 0xff] ^ tables.t[6][(lo >> 8) & 0xff] ^ tables.t[5][(lo >> 16) & 0xff] ^
              tables.t[4][lo >> 24] ^ tables.t[3][hi & 0xff] ^ tables.t[2][(hi >> 8) & 0xff] ^
              tables.t[1][(hi >> 16) & 0xff] ^ tables.t[0][hi >> 24];
        p += 8, size -= 8;
    }
    while (size--)
        crc = (crc >> 8) ^ tables.t[0][(crc ^ *p++) & 0xff];
    return ~crc;
}

[[noreturn]] void fail(const std::string &what) {
    throw std::runtime_error("checkpoint: " + what);
}

// ---- little-endian byte buffers --------------------------------------------------------------
struct Bytes {
    std::vector<unsigned char> data;
    void u8(unsigned v) { data.push_back(static_cast<unsigned char>(v)); }
    void u16(unsigned v) { u8(v & 0xff), u8((v >> 8) & 0xff); }
    void u32(uint32_t v) { u16(v & 0xffff), u16(v >> 16); }
    void u64(uint64_t v) { u32(uint32_t(v)), u32(uint32_t(v >> 32)); }
    void text(const std::string &s) { data.insert(data.end(), s.begin(), s.end()); }
};
uint64_t le(const unsigned char *p, int bytes) {
    uint64_t v = 0;
    for (int i = bytes - 1; i >= 0; --i)
        v = (v << 8) | p[i];
    return v;
}

// ---- the pickle ----------------------------------------------------------------------------------
enum Kind { LONG = 0, FLOAT = 1, DOUBLE = 2 };
const char *const STORAGE_CLASS[] = {"LongStorage", "FloatStorage", "DoubleStorage"};
const int ELEMENT_BYTES[] = {8, 4, 8};

struct Pickle : Bytes {
    void str(const std::string &s) { u8('X'), u32(uint32_t(s.size())), text(s); }          // BINUNICODE
    void global(const char *module, const char *name) { u8('c'), text(module), u8('\n'), text(name), u8('\n'); }
    void integer(int64_t v) {                                                                // BININT / LONG1
        if (v >= INT32_MIN && v <= INT32_MAX) {
            u8('J'), u32(uint32_t(int32_t(v)));
        } else {
            u8(0x8a), u8(8), u64(uint64_t(v));
        }
    }
    // key -> 1-D tensor of `count` elements backed by storage `storage`
    void tensor(const char *key, Kind kind, int storage, int64_t count) {
        str(key);
        global("torch._utils", "_rebuild_tensor_v2");
        u8('(');                                             // MARK: arguments of _rebuild_tensor_v2
        u8('('), str("storage"), global("torch", STORAGE_CLASS[kind]), str(std::to_string(storage)), str("cpu");
        integer(count), u8('t'), u8('Q');                    // TUPLE, BINPERSID
        u8('K'), u8(0);                                      // storage offset
        integer(count), u8(0x85);                            // size  (TUPLE1)
        u8('K'), u8(1), u8(0x85);                            // stride
        u8(0x89);                                            // requires_grad = False
        global("collections", "OrderedDict"), u8(')'), u8('R'); // backward hooks = OrderedDict()
        u8('t'), u8('R');                                    // TUPLE, REDUCE
    }
    void open(const char *key) { str(key), u8('}'), u8('('); } // key -> EMPTY_DICT, MARK
    void close() { u8('u'); }                                    // SETITEMS
};

struct Storage {
    Kind kind;
    int64_t count;
    const void *data; // writing
    void *out;        // reading
};
enum {
    S_DEPTH, S_CONTEXT, S_WEIGHTS, S_MOMENTUM, S_VARIANCE, S_STEP, S_TOTAL_STEPS, S_WARMUP, S_INITIAL, S_FINAL,
    S_LOW, S_HIGH, S_SECONDS, S_LOSS_SUMS, S_LOSS_BATCHES, S_D_MODEL, S_HEADS, S_VOCAB, S_FFN, STORAGES
};

Pickle make_pickle(int64_t parameters, int64_t loss_positions) {
    Pickle p;
    p.u8(0x80), p.u8(2), p.u8('}'), p.u8('(');
    p.open("model");
    p.tensor("depth", LONG, S_DEPTH, 1), p.tensor("context", LONG, S_CONTEXT, 1);
    p.tensor("weights", FLOAT, S_WEIGHTS, parameters);
    p.tensor("d_model", LONG, S_D_MODEL, 1), p.tensor("heads", LONG, S_HEADS, 1);
    p.tensor("vocab", LONG, S_VOCAB, 1), p.tensor("ffn", LONG, S_FFN, 1);
    p.close();
    p.open("opt");
    p.tensor("momentum", FLOAT, S_MOMENTUM, parameters), p.tensor("variance", FLOAT, S_VARIANCE, parameters);
    p.tensor("step", LONG, S_STEP, 1);
    p.close();
    p.open("lr_scheduler");
    p.tensor("total_steps", LONG, S_TOTAL_STEPS, 1), p.tensor("step", LONG, S_STEP, 1);
    p.tensor("warmup_fraction", DOUBLE, S_WARMUP, 1), p.tensor("initial_lr_fraction", DOUBLE, S_INITIAL, 1);
    p.tensor("final_lr_fraction", DOUBLE, S_FINAL, 1), p.tensor("low_momentum", DOUBLE, S_LOW, 1);
    p.tensor("high_momentum", DOUBLE, S_HIGH, 1);
    p.close();
    p.open("trainer");
    p.tensor("train_seconds", DOUBLE, S_SECONDS, 1), p.tensor("final_loss_sums", DOUBLE, S_LOSS_SUMS, loss_positions);
    p.tensor("final_loss_batches", LONG, S_LOSS_BATCHES, 1);
    p.close();
    p.close(), p.u8('.');
    return p;
}

// ---- ZIP writer (stored records, 64-byte aligned payloads, zip64 end records) -----------------------
constexpr uint32_t SIG_LOCAL = 0x04034b50, SIG_CENTRAL = 0x02014b50, SIG_END = 0x06054b50,
                   SIG_END64 = 0x06064b50, SIG_LOCATOR64 = 0x07064b50;
const char *const PREFIX = "archive";
// the record the reference's reader insists on (checkpoint.cpp:15): 40 characters
const char *const SERIALIZATION_ID = "3407000000000000000000000000000000000000";
constexpr uint64_t CHECKPOINT_LIMIT = 0xffffffffull; // sizes and offsets are 32-bit fields

struct FileCloser {
    void operator()(FILE *f) const {
        if (f)
            std::fclose(f);
    }
};
using File = std::unique_ptr<FILE, FileCloser>;

class ZipWriter {
  public:
    explicit ZipWriter(FILE *file) : file_(file) {}
    void add(const std::string &name, const void *data, uint64_t size) {
        if (size >= 0xffffffffull || offset_ >= 0xffffffffull)
            fail("record " + name + " does not fit the 32-bit ZIP fields");
        const uint32_t crc = crc32_of(data, size_t(size));
        // pad with an extra field so that the payload starts on a 64-byte boundary
        const uint64_t after_name = offset_ + 30 + name.size();
        unsigned extra = unsigned(64 - (after_name + 4) % 64) % 64 + 4;
        Bytes h;
        h.u32(SIG_LOCAL), h.u16(20), h.u16(0), h.u16(0), h.u16(0), h.u16(0);
        h.u32(crc), h.u32(uint32_t(size)), h.u32(uint32_t(size));
        h.u16(unsigned(name.size())), h.u16(extra), h.text(name);
        h.u16(0x4246), h.u16(extra - 4);
        h.data.insert(h.data.end(), extra - 4, 'Z');
        entries_.push_back({name, crc, uint32_t(size), uint32_t(offset_)});
        put(h.data.data(), h.data.size());
        put(data, size_t(size));
    }
    void add(const std::string &name, const std::string &text) { add(name, text.data(), text.size()); }
    void finish() {
        const uint64_t central = offset_;
        for (const Entry &e : entries_) {
            Bytes c;
            c.u32(SIG_CENTRAL), c.u16(20), c.u16(20), c.u16(0), c.u16(0), c.u16(0), c.u16(0);
            c.u32(e.crc), c.u32(e.size), c.u32(e.size);
            c.u16(unsigned(e.name.size())), c.u16(0), c.u16(0), c.u16(0), c.u16(0), c.u32(0), c.u32(e.offset);
            c.text(e.name);
            put(c.data.data(), c.data.size());
        }
        const uint64_t central_size = offset_ - central, end64 = offset_;
        Bytes t;
        t.u32(SIG_END64), t.u64(44), t.u16(20), t.u16(20), t.u32(0), t.u32(0);
        t.u64(entries_.size()), t.u64(entries_.size()), t.u64(central_size), t.u64(central);
        t.u32(SIG_LOCATOR64), t.u32(0), t.u64(end64), t.u32(1);
        t.u32(SIG_END), t.u16(0), t.u16(0), t.u16(unsigned(entries_.size())), t.u16(unsigned(entries_.size()));
        t.u32(uint32_t(central_size)), t.u32(uint32_t(central)), t.u16(0);
        put(t.data.data(), t.data.size());
    }

  private:
    struct Entry {
        std::string name;
        uint32_t crc, size, offset;
    };
    void put(const void *data, size_t size) {
        if (size && std::fwrite(data, 1, size, file_) != size)
            fail(std::string("write failed: ") + std::strerror(errno));
        offset_ += size;
    }
    FILE *file_;
    uint64_t offset_ = 0;
    std::vector<Entry> entries_;
};

// ---- ZIP reader --------------------------------------------------------------------------------
struct Record {
    uint64_t offset; // of the payload
    uint32_t size, crc;
};
class ZipReader {
  public:
    explicit ZipReader(const char *path) : file_(std::fopen(path, "rb")) {
        if (!file_)
            fail(std::string("cannot open ") + path + ": " + std::strerror(errno));
        std::fseek(file_.get(), 0, SEEK_END);
        size_ = uint64_t(std::ftell(file_.get()));
        if (size_ < 22)
            fail("truncated file");
        // end-of-central-directory record: search the last 64 KiB + 22 bytes backwards
        const uint64_t window = size_ < 65557 ? size_ : 65557;
        std::vector<unsigned char> tail = read_at(size_ - window, size_t(window));
        int64_t at = int64_t(window) - 22;
        while (at >= 0 && le(&tail[size_t(at)], 4) != SIG_END)
            --at;
        if (at < 0)
            fail("no ZIP end record");
        uint64_t count = le(&tail[size_t(at) + 10], 2), central_size = le(&tail[size_t(at) + 12], 4),
                 central = le(&tail[size_t(at) + 16], 4);
        if (at >= 20 && le(&tail[size_t(at) - 20], 4) == SIG_LOCATOR64) {
            const uint64_t end64 = le(&tail[size_t(at) - 12], 8);
            const std::vector<unsigned char> r = read_at(end64, 56);
            if (le(r.data(), 4) != SIG_END64)
                fail("bad zip64 end record");
            count = le(&r[32], 8), central_size = le(&r[40], 8), central = le(&r[48], 8);
        }
        if (central + central_size > size_)
            fail("central directory out of range");
        const std::vector<unsigned char> dir = read_at(central, size_t(central_size));
        size_t p = 0;
        for (uint64_t i = 0; i < count; ++i) {
            if (p + 46 > dir.size() || le(&dir[p], 4) != SIG_CENTRAL)
                fail("bad central directory entry");
            const unsigned method = unsigned(le(&dir[p + 10], 2));
            const uint32_t crc = uint32_t(le(&dir[p + 16], 4)), packed = uint32_t(le(&dir[p + 20], 4)),
                           size = uint32_t(le(&dir[p + 24], 4));
            const size_t name_len = size_t(le(&dir[p + 28], 2)), extra = size_t(le(&dir[p + 30], 2)),
                         comment = size_t(le(&dir[p + 32], 2));
            const uint64_t local = le(&dir[p + 42], 4);
            if (p + 46 + name_len > dir.size())
                fail("bad central directory entry");
            const std::string name(reinterpret_cast<const char *>(&dir[p + 46]), name_len);
            if (method != 0 || packed != size)
                fail("record " + name + " is compressed");
            const std::vector<unsigned char> lh = read_at(local, 30);
            if (le(lh.data(), 4) != SIG_LOCAL)
                fail("bad local header of " + name);
            const uint64_t payload = local + 30 + le(&lh[26], 2) + le(&lh[28], 2);
            if (payload + size > size_)
                fail("record " + name + " is truncated");
            if (!records_.emplace(name, Record{payload, size, crc}).second)
                fail("duplicate record " + name);
            p += 46 + name_len + extra + comment;
        }
    }
    bool has(const std::string &name) const { return records_.count(name) != 0; }
    const Record &find(const std::string &name) const {
        const auto it = records_.find(name);
        if (it == records_.end())
            fail("missing record " + name);
        return it->second;
    }
    // the directory prefix: the one record called <prefix>/data.pkl
    std::string prefix() const {
        for (const auto &r : records_) {
            const std::string &n = r.first;
            if (n.size() > 9 && n.compare(n.size() - 9, 9, "/data.pkl") == 0)
                return n.substr(0, n.size() - 9);
        }
        fail("missing data.pkl");
    }
    // payload of a record, CRC checked; into `out` (exactly `bytes` long)
    void load(const std::string &name, void *out, uint64_t bytes) const {
        const Record &r = find(name);
        if (r.size != bytes)
            fail("record " + name + " has " + std::to_string(r.size) + " bytes, expected " + std::to_string(bytes));
        std::fseek(file_.get(), long(r.offset), SEEK_SET);
        if (bytes && std::fread(out, 1, size_t(bytes), file_.get()) != bytes)
            fail("cannot read record " + name);
        if (crc32_of(out, size_t(bytes)) != r.crc)
            fail("CRC mismatch in record " + name);
    }
    std::string text(const std::string &name) const {
        const Record &r = find(name);
        std::string s(r.size, '\0');
        load(name, &s[0], r.size);
        return s;
    }

  private:
    std::vector<unsigned char> read_at(uint64_t offset, size_t bytes) const {
        std::vector<unsigned char> out(bytes);
        if (offset + bytes > size_ || std::fseek(file_.get(), long(offset), SEEK_SET) != 0 ||
            (bytes && std::fread(out.data(), 1, bytes, file_.get()) != bytes))
            fail("truncated file");
        return out;
    }
    File file_;
    uint64_t size_ = 0;
    std::map<std::string, Record> records_;
};

// ---- the checkpoint <-> its storages ------------------------------------------------------------------
struct Scalars {
    int64_t depth, context, step, total_steps, loss_batches, d_model, heads, vocab, ffn;
    double warmup, initial, final_fraction, low, high, seconds;
};
std::string record_name(const std::string &prefix, int storage) {
    return prefix + "/data/" + std::to_string(storage);
}

// Elements of weights / momentum / variance.  Width 16 with 4 heads and a 48-wide MLP is the reference's own
// network, whose flat layout is model.h:12-37 (no positions, no biases); every other shape is the wide
// model of include/tg_model.h.
int64_t expected_parameters(const TgModelConfig &m) {
    if (m.d_model == 16 && m.heads == 4 && m.vocab == 256 && m.ffn == 48)
        return 2 * 256 * 16 + 16 + int64_t(m.base.depth) * (2 * 16 + 4 * 48 * 16 + 16 * 16);
    return tg_parameter_layout(&m).count;
}

void check_for_writing(const TgCheckpoint &c) {
    const TgModelConfig &m = c.model;
    if (m.base.depth < 1 || m.base.context < 1 || m.d_model < 1 || m.heads < 1 || m.vocab < 1 || m.ffn < 1)
        fail("model fields must be positive");
    const int64_t expected = m.base.depth > TG_MAX_DEPTH ? -1 : expected_parameters(m);
    if (expected != c.parameter_count)
        fail("parameter_count " + std::to_string(c.parameter_count) + " does not match the model (" +
             std::to_string(expected) + ")");
    if (!c.weights || !c.momentum || !c.variance)
        fail("weights, momentum and variance are required");
    if (c.final_loss_positions != 0 && c.final_loss_positions != m.base.context)
        fail("final_loss_positions must be 0 or the context length");
    if (c.final_loss_positions && !c.final_loss_sums)
        fail("final_loss_sums is missing");
    if (c.scheduler.total_steps < 0)
        fail("scheduler.total_steps is negative");
    // A width-16 file is promised to load through the reference's load_training_state, which refuses what follows
    // (checkpoint.cpp:535-550, optim.h:18-30): such a state is refused here, before anything is written.
    if (m.d_model == 16 && m.heads == 4 && m.vocab == 256 && m.ffn == 48) {
        const OneCycle &s = c.scheduler;
        if (c.final_loss_positions != m.base.context)
            fail("a width-16 checkpoint carries one final-loss sum per position (final_loss_positions = context)");
        if (s.total_steps < 1 || c.step > uint64_t(s.total_steps))
            fail("a width-16 checkpoint needs scheduler.total_steps >= 1 and step <= total_steps");
        const int64_t total = s.total_steps, window = std::max<int64_t>(1, (total + 99) / 100);
        const int64_t first = std::max<int64_t>(0, total - window);
        if (int64_t(c.final_loss_batches) > std::max<int64_t>(0, int64_t(c.step) - first))
            fail("final_loss_batches exceeds the steps of the final-loss window that have run");
        const bool fractions = s.warmup_fraction > 0 && s.warmup_fraction < 1 && s.initial_lr_fraction > 0 &&
                               s.initial_lr_fraction < 1 && s.final_lr_fraction > 0 &&
                               s.final_lr_fraction <= s.initial_lr_fraction && s.low_momentum >= 0 && s.low_momentum < 1 &&
                               s.high_momentum >= s.low_momentum && s.high_momentum < 1;
        if (!fractions || s.warmup_fraction * s.total_steps - 1 == 0)
            fail("a width-16 checkpoint needs a valid OneCycle schedule");
    }
}

void write_checkpoint(const char *path, const TgCheckpoint &c) {
    check_for_writing(c);
    const Scalars s = {c.model.base.depth, c.model.base.context, int64_t(c.step), c.scheduler.total_steps,
                       int64_t(c.final_loss_batches), c.model.d_model, c.model.heads, c.model.vocab, c.model.ffn,
                       c.scheduler.warmup_fraction, c.scheduler.initial_lr_fraction, c.scheduler.final_lr_fraction,
                       c.scheduler.low_momentum, c.scheduler.high_momentum, c.train_seconds};
    const Storage storages[STORAGES] = {
        {LONG, 1, &s.depth, nullptr},       {LONG, 1, &s.context, nullptr},
        {FLOAT, c.parameter_count, c.weights, nullptr},
        {FLOAT, c.parameter_count, c.momentum, nullptr},
        {FLOAT, c.parameter_count, c.variance, nullptr},
        {LONG, 1, &s.step, nullptr},        {LONG, 1, &s.total_steps, nullptr},
        {DOUBLE, 1, &s.warmup, nullptr},    {DOUBLE, 1, &s.initial, nullptr},
        {DOUBLE, 1, &s.final_fraction, nullptr}, {DOUBLE, 1, &s.low, nullptr},
        {DOUBLE, 1, &s.high, nullptr},      {DOUBLE, 1, &s.seconds, nullptr},
        {DOUBLE, c.final_loss_positions, c.final_loss_sums, nullptr},
        {LONG, 1, &s.loss_batches, nullptr}, {LONG, 1, &s.d_model, nullptr},
        {LONG, 1, &s.heads, nullptr},       {LONG, 1, &s.vocab, nullptr},
        {LONG, 1, &s.ffn, nullptr}};
    // every record and the archive as a whole must fit the 32-bit ZIP fields the reference's reader uses
    // (checkpoint.cpp:386-411): refuse before anything is written
    uint64_t total = 1 << 16; // headers, pickle and directory
    for (int i = 0; i < STORAGES; ++i) {
        const uint64_t bytes = uint64_t(storages[i].count) * ELEMENT_BYTES[storages[i].kind];
        if (bytes >= CHECKPOINT_LIMIT)
            fail("an array of " + std::to_string(bytes) + " bytes does not fit a checkpoint (limit 4 GiB per file)");
        total += bytes + 256;
    }
    if (total >= CHECKPOINT_LIMIT)
        fail("the model's state (" + std::to_string(total) + " bytes) does not fit a checkpoint (limit 4 GiB per file)");
    const std::string temporary = std::string(path) + ".tmp";
    try {
        File file(std::fopen(temporary.c_str(), "wb"));
        if (!file)
            fail("cannot create " + temporary + ": " + std::strerror(errno));
        ZipWriter zip(file.get());
        const Pickle pickle = make_pickle(c.parameter_count, c.final_loss_positions);
        const std::string prefix = PREFIX;
        zip.add(prefix + "/data.pkl", pickle.data.data(), pickle.data.size());
        zip.add(prefix + "/.format_version", "2");
        zip.add(prefix + "/.storage_alignment", "64");
        zip.add(prefix + "/byteorder", "little");
        for (int i = 0; i < STORAGES; ++i)
            zip.add(record_name(prefix, i), storages[i].data, uint64_t(storages[i].count) * ELEMENT_BYTES[storages[i].kind]);
        zip.add(prefix + "/version", "3\n");
        zip.add(prefix + "/.data/serialization_id", SERIALIZATION_ID); // checkpoint.cpp:15,323,519-524
        zip.finish();
        if (std::fflush(file.get()) != 0)
            fail(std::string("write failed: ") + std::strerror(errno));
    } catch (...) {
        std::remove(temporary.c_str()); // no partial file stays behind, whatever failed
        throw;
    }
    if (std::rename(temporary.c_str(), path) != 0) {
        const std::string why = std::strerror(errno);
        std::remove(temporary.c_str());
        fail(std::string("cannot replace ") + path + ": " + why);
    }
}

// scalars, container metadata and counts; returns the prefix
std::string read_header(const ZipReader &zip, TgCheckpoint &c) {
    const std::string prefix = zip.prefix();
    if (zip.text(prefix + "/.format_version") != "2" || zip.text(prefix + "/byteorder") != "little" ||
        zip.text(prefix + "/version") != "3\n")
        fail("unsupported container metadata");
    Scalars s{};
    const struct {
        int storage;
        void *out;
    } scalars[] = {{S_DEPTH, &s.depth},       {S_CONTEXT, &s.context},   {S_STEP, &s.step},
                   {S_TOTAL_STEPS, &s.total_steps}, {S_LOSS_BATCHES, &s.loss_batches},
                   {S_WARMUP, &s.warmup},     {S_INITIAL, &s.initial},   {S_FINAL, &s.final_fraction},
                   {S_LOW, &s.low},           {S_HIGH, &s.high},         {S_SECONDS, &s.seconds}};
    for (const auto &item : scalars)
        zip.load(record_name(prefix, item.storage), item.out, 8);
    // The width fields are this library's addition (storages 15 .. 18).  A file the reference wrote has
    // storages 0 .. 14 only and holds the reference's own network: width 16, 4 heads, vocabulary 256, MLP 48.
    if (zip.has(record_name(prefix, S_D_MODEL))) {
        zip.load(record_name(prefix, S_D_MODEL), &s.d_model, 8), zip.load(record_name(prefix, S_HEADS), &s.heads, 8);
        zip.load(record_name(prefix, S_VOCAB), &s.vocab, 8), zip.load(record_name(prefix, S_FFN), &s.ffn, 8);
    } else {
        s.d_model = 16, s.heads = 4, s.vocab = 256, s.ffn = 48;
    }
    if (s.depth < 1 || s.depth > TG_MAX_DEPTH || s.context < 1 || s.context > (1 << 24) || s.d_model < 1 ||
        s.d_model > (1 << 20) || s.heads < 1 || s.vocab < 1 || s.vocab > (1 << 24) || s.ffn < 1 || s.ffn > (1 << 24) ||
        s.step < 0 || s.total_steps < 0 || s.total_steps > INT32_MAX || s.loss_batches < 0)
        fail("architecture or counter fields out of range");
    std::memset(&c.model, 0, sizeof c.model);
    c.model.base.depth = int(s.depth), c.model.base.context = int(s.context);
    c.model.d_model = int(s.d_model), c.model.heads = int(s.heads), c.model.vocab = int(s.vocab), c.model.ffn = int(s.ffn);
    c.parameter_count = expected_parameters(c.model);
    if (zip.find(record_name(prefix, S_WEIGHTS)).size != uint64_t(c.parameter_count) * 4 ||
        zip.find(record_name(prefix, S_MOMENTUM)).size != uint64_t(c.parameter_count) * 4 ||
        zip.find(record_name(prefix, S_VARIANCE)).size != uint64_t(c.parameter_count) * 4)
        fail("state arrays do not match the model");
    const uint32_t loss_bytes = zip.find(record_name(prefix, S_LOSS_SUMS)).size;
    if (loss_bytes != 0 && loss_bytes != uint64_t(s.context) * 8)
        fail("final loss state does not match the model");
    c.final_loss_positions = loss_bytes / 8;
    c.step = uint64_t(s.step);
    c.scheduler = OneCycle{int(s.total_steps), s.warmup, s.initial, s.final_fraction, s.low, s.high};
    c.train_seconds = s.seconds;
    c.final_loss_batches = uint64_t(s.loss_batches);
    return prefix;
}

} // namespace

TG_API int tg_checkpoint_write(const char *path, const TgCheckpoint *checkpoint) {
    return guarded([&] {
        require(path && checkpoint, "checkpoint: missing argument");
        write_checkpoint(path, *checkpoint);
    });
}

TG_API int tg_checkpoint_inspect(const char *path, TgCheckpoint *header) {
    return guarded([&] {
        require(path && header, "checkpoint: missing argument");
        TgCheckpoint found = *header;
        const ZipReader zip(path);
        read_header(zip, found);
        found.weights = header->weights, found.momentum = header->momentum, found.variance = header->variance;
        found.final_loss_sums = header->final_loss_sums;
        *header = found;
    });
}

TG_API int tg_checkpoint_read(const char *path, TgCheckpoint *checkpoint) {
    return guarded([&] {
        require(path && checkpoint, "checkpoint: missing argument");
        TgCheckpoint found = *checkpoint;
        const ZipReader zip(path);
        const std::string prefix = read_header(zip, found);
        const TgModelConfig &want = checkpoint->model, &have = found.model;
        if (want.d_model != 0 &&
            (want.base.depth != have.base.depth || want.base.context != have.base.context ||
             want.d_model != have.d_model || want.heads != have.heads || want.vocab != have.vocab ||
             want.ffn != have.ffn))
            fail("architecture mismatch");
        if (checkpoint->parameter_count != found.parameter_count ||
            checkpoint->final_loss_positions != found.final_loss_positions)
            fail("buffer sizes differ from the file's (see tg_checkpoint_inspect)");
        require(checkpoint->weights && checkpoint->momentum && checkpoint->variance &&
                    (found.final_loss_positions == 0 || checkpoint->final_loss_sums),
                "checkpoint: missing output buffer");
        zip.load(record_name(prefix, S_WEIGHTS), checkpoint->weights, uint64_t(found.parameter_count) * 4);
        zip.load(record_name(prefix, S_MOMENTUM), checkpoint->momentum, uint64_t(found.parameter_count) * 4);
        zip.load(record_name(prefix, S_VARIANCE), checkpoint->variance, uint64_t(found.parameter_count) * 4);
        zip.load(record_name(prefix, S_LOSS_SUMS), checkpoint->final_loss_sums, uint64_t(found.final_loss_positions) * 8);
        found.weights = checkpoint->weights, found.momentum = checkpoint->momentum;
        found.variance = checkpoint->variance, found.final_loss_sums = checkpoint->final_loss_sums;
        *checkpoint = found;
    });
}

// The loss summary a run carries through its checkpoints (loss_summary.cpp:5-29): per-position sums over the
// steps after total_steps - max(1, ceil(total_steps / 100)).
TG_API int tg_final_loss_add(int total_steps, int positions, int completed_step, const float *losses, double *sums,
                             uint64_t *batches) {
    return guarded([&] {
        require(total_steps >= 0 && positions > 0 && losses && sums && batches, "final loss: missing argument");
        const int window = (total_steps + 99) / 100 > 1 ? (total_steps + 99) / 100 : 1;
        const int first_step = total_steps > window ? total_steps - window : 0;
        if (completed_step <= first_step)
            return;
        for (int p = 0; p < positions; ++p)
            sums[p] += losses[p];
        ++*batches;
    });
}
