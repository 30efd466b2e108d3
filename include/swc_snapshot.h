/*
 * swc_snapshot.h — snapshots of a training program: the trained tensors and
 * the iteration count, written every TrainingConfig::snapshot iterations to
 * "snapshot_iter<N>.model" and read back when the program is started with
 * --snapshot=<file>.
 *
 * The file is the reference's: a serialized caffe2 NetDef with one OperatorDef
 * per tensor (its `name` is the tensor's variable name, its first Argument is
 * called "values" and carries the elements as `floats`) and one NetDef-level
 * Argument "iter" (reference: src/codegen/utils/utils.h:5-68, written and read
 * by the code of src/codegen/Codegen.cpp:659-812).  The reference goes through
 * libprotobuf; this header writes and reads the wire format of those few
 * fields itself (caffe2.proto: NetDef.op = 2, NetDef.arg = 6, OperatorDef.name
 * = 3, OperatorDef.arg = 5, Argument.name = 1, Argument.i = 3, Argument.floats
 * = 5), in the field order protobuf serializes them, so a file of either
 * program restores the other.  Function names are the reference's (addOp,
 * loadFromSnapShot, getIterFromSnapShot) so that generated call sites read the
 * same.
 */
#ifndef SWC_SNAPSHOT_H_
#define SWC_SNAPSHOT_H_

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <string>
#include <vector>

class SnapshotNet {
  public:
    // ---- writing: tensors are appended to the serialized form as they come
    void addTensor(const std::string &name, const float *var, size_t size) {
        // Argument{name="values", floats=...}: each element is a tag byte and four value bytes (proto2 repeated
        // fields are not packed unless declared so)
        const std::string argName = "values";
        const uint64_t argLen = 1 + varintLen(argName.size()) + argName.size() + 5 * (uint64_t)size;
        const uint64_t opLen = 1 + varintLen(name.size()) + name.size() + 1 + varintLen(argLen) + argLen;
        out_.reserve(out_.size() + (size_t)opLen + 16);
        putTag(2, 2), putVarint(opLen);
        putTag(3, 2), putVarint(name.size()), out_ += name;
        putTag(5, 2), putVarint(argLen);
        putTag(1, 2), putVarint(argName.size()), out_ += argName;
        for (size_t i = 0; i < size; ++i) {
            uint32_t bits;
            std::memcpy(&bits, var + i, 4);
            const char b[5] = {(char)0x2D, (char)(bits & 0xff), (char)(bits >> 8 & 0xff), (char)(bits >> 16 & 0xff),
                               (char)(bits >> 24 & 0xff)};
            out_.append(b, 5);
        }
    }
    void setIter(uint64_t iter) { iter_ = iter, has_iter_ = true; }
    bool save(const std::string &path) const {
        std::string tail;   // NetDef.arg follows every NetDef.op
        if (has_iter_) {
            SnapshotNet a;
            const std::string argName = "iter";
            a.putTag(1, 2), a.putVarint(argName.size()), a.out_ += argName;
            a.putTag(3, 0), a.putVarint(iter_);
            SnapshotNet t;
            t.putTag(6, 2), t.putVarint(a.out_.size());
            tail = t.out_ + a.out_;
        }
        std::FILE *f = std::fopen(path.c_str(), "wb");
        if (!f) return false;
        const bool ok = std::fwrite(out_.data(), 1, out_.size(), f) == out_.size() &&
                        std::fwrite(tail.data(), 1, tail.size(), f) == tail.size();
        return std::fclose(f) == 0 && ok;
    }

    // ---- reading: the file is kept as it is, with an index of where each tensor's elements lie
    bool parse(const std::string &path) {
        std::FILE *f = std::fopen(path.c_str(), "rb");
        if (!f) return false;
        std::fseek(f, 0, SEEK_END);
        const long n = std::ftell(f);
        std::rewind(f);
        in_.resize(n > 0 ? (size_t)n : 0);
        const bool ok = std::fread(&in_[0], 1, in_.size(), f) == in_.size();
        std::fclose(f);
        return ok && parseNet(0, in_.size());
    }
    // the elements of tensor `name` -> var; false if the snapshot has no such tensor.  A tensor of another size
    // means a snapshot of another model: that ends the program.
    bool restore(const std::string &name, float *var, size_t size) const {
        for (const Entry &e : entries_) {
            if (e.name != name) continue;
            size_t k = 0;
            bool fits = true;
            for (const Span &s : e.floats)
                for (size_t p = s.begin; p + 4 <= s.end && fits; p += 4) {
                    if (k == size) {
                        fits = false;
                        break;
                    }
                    std::memcpy(var + k++, &in_[p], 4);   // (little-endian hosts, like the tensor files)
                }
            if (!fits || k != size) {
                std::cout << "snapshot tensor " << name << " does not have " << size << " elements\n";
                std::exit(EXIT_FAILURE);
            }
            return true;
        }
        return false;
    }
    size_t iter() const { return (size_t)iter_; }
    size_t tensors() const { return entries_.size(); }

  private:
    struct Span {
        size_t begin, end;
    };
    struct Entry {
        std::string name;
        std::vector<Span> floats;   // byte ranges of 4-byte elements, in order
    };
    std::string out_, in_;
    std::vector<Entry> entries_;
    uint64_t iter_{0};
    bool has_iter_{false};

    static size_t varintLen(uint64_t v) {
        size_t n = 1;
        while (v >= 0x80) v >>= 7, ++n;
        return n;
    }
    void putVarint(uint64_t v) {
        while (v >= 0x80) out_ += (char)(v | 0x80), v >>= 7;
        out_ += (char)v;
    }
    void putTag(unsigned field, unsigned wire) { putVarint(field << 3 | wire); }

    bool getVarint(size_t &p, size_t end, uint64_t &v) const {
        v = 0;
        for (int shift = 0; shift < 64 && p < end; shift += 7) {
            const unsigned char b = (unsigned char)in_[p++];
            v |= (uint64_t)(b & 0x7f) << shift;
            if (!(b & 0x80)) return true;
        }
        return false;
    }
    // one field: its number, wire type and payload range [begin,end) (varints: the value in `v`)
    bool getField(size_t &p, size_t end, unsigned &field, unsigned &wire, size_t &begin, size_t &fend, uint64_t &v) const {
        uint64_t key;
        if (!getVarint(p, end, key)) return false;
        field = (unsigned)(key >> 3), wire = (unsigned)(key & 7);
        v = 0;
        if (wire == 0) {
            begin = p;
            if (!getVarint(p, end, v)) return false;
        } else if (wire == 1 || wire == 5) {
            begin = p;
            p += wire == 1 ? 8 : 4;
        } else if (wire == 2) {
            uint64_t len;
            if (!getVarint(p, end, len) || len > end - p) return false;
            begin = p;
            p += (size_t)len;
        } else {
            return false;   // groups do not occur in these messages
        }
        fend = p;
        return p <= end;
    }
    bool parseNet(size_t p, size_t end) {
        unsigned field, wire;
        size_t b, e;
        uint64_t v;
        while (p < end) {
            if (!getField(p, end, field, wire, b, e, v)) return false;
            if (field == 2 && wire == 2) {
                Entry entry;
                if (!parseOp(b, e, entry)) return false;
                entries_.push_back(entry);
            } else if (field == 6 && wire == 2) {
                std::string name;
                uint64_t i = 0;
                std::vector<Span> none;
                if (!parseArg(b, e, name, i, none)) return false;
                if (name == "iter") iter_ = i, has_iter_ = true;
            }
        }
        return true;
    }
    bool parseOp(size_t p, size_t end, Entry &entry) const {
        unsigned field, wire;
        size_t b, e;
        uint64_t v;
        bool first = true;
        while (p < end) {
            if (!getField(p, end, field, wire, b, e, v)) return false;
            if (field == 3 && wire == 2) entry.name.assign(in_, b, e - b);
            if (field == 5 && wire == 2 && first) {   // the reference reads arg(0), whatever it is called
                std::string name;
                uint64_t i;
                if (!parseArg(b, e, name, i, entry.floats)) return false;
                first = false;
            }
        }
        return true;
    }
    bool parseArg(size_t p, size_t end, std::string &name, uint64_t &i, std::vector<Span> &floats) const {
        unsigned field, wire;
        size_t b, e;
        uint64_t v;
        while (p < end) {
            if (!getField(p, end, field, wire, b, e, v)) return false;
            if (field == 1 && wire == 2) name.assign(in_, b, e - b);
            if (field == 3 && wire == 0) i = v;
            if (field == 5 && (wire == 5 || wire == 2)) {   // one element, or a packed run of them
                if (!floats.empty() && floats.back().end == b) floats.back().end = e;
                else floats.push_back(Span{b, e});
            }
        }
        return true;
    }
};

// the reference's names (src/codegen/utils/utils.h:23-68)
inline void addOp(SnapshotNet &net, const std::string &name, const float *var, size_t size) { net.addTensor(name, var, size); }
inline bool loadFromSnapShot(const SnapshotNet &net, const std::string &name, float *var, size_t size) {
    if (net.restore(name, var, size)) return true;
    std::cerr << "snapshot has no tensor " << name << ": it keeps its initial value\n";
    return false;
}
inline size_t getIterFromSnapShot(const SnapshotNet &net) { return net.iter(); }

// Value of the command-line flag `name`, written --name=value, -name=value, --name value or -name value (the
// spellings the reference's gflags accepts); "" if it is not given.
inline std::string swcFlagString(int argc, char **argv, const char *name) {
    const std::string key(name);
    for (int a = 1; a < argc; ++a) {
        std::string s(argv[a]);
        if (s.size() < 2 || s[0] != '-') continue;
        s.erase(0, s[1] == '-' ? 2 : 1);
        if (s == key) return a + 1 < argc ? std::string(argv[a + 1]) : std::string();
        if (s.compare(0, key.size() + 1, key + "=") == 0) return s.substr(key.size() + 1);
    }
    return std::string();
}

#endif /* SWC_SNAPSHOT_H_ */
