// The .nc data path: NetCDF-3 classic reader and fraction builder (host code only).
//
// Reference behaviour: data_sets/DataSet.cpp
//   :60-195      helpers around libnetcdf (dimension lookup, string / int / pattern arrays)
//   :1376-1500   per file: dimensions, fraction of the sequences, truncation into segments
//   :1500-1840   per segment: inputs / targetPatterns / targetClasses rows [begin, begin + length)
//   :1897-1900   training mode: sequences sorted by ascending length
//   :642-1022    _makeFractionTask: S parallel sequences interleaved time-major, patTypes, targets
// File format: README section 5 of the reference (dimensions numSeqs, numTimesteps, inputPattSize,
// targetPattSize | numLabels, maxSeqTagLength; variables seqTags, seqLengths, inputs, targetPatterns |
// targetClasses), written by its tooling with scipy's netcdf_file (pyTools/dataTools/ncDataHandle.py:174-186).
//
// libnetcdf is not used: the classic format (CDF-1) and its 64-bit-offset variant (CDF-2) are a flat
// big-endian header followed by the variables' row-major data, parsed here.  Record (unlimited-dimension)
// variables are refused with a clear message.  The reference copies every sequence into a cache file under
// /tmp first and builds fractions from there; here a fraction is built straight from the .nc file with one
// positioned read per sequence and variable.
// Not covered (refused or absent): several .nc files in one set, input context windows and output time lag,
// noise injection, external / auxiliary data, sequence and fraction shuffling, ordered file lists.
#include "common.hpp"

#include <random>
#include <algorithm>
#include <cerrno>
#include <cstring>
#include <limits>
#include <new>
#include <string>
#include <vector>

#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

namespace cnt {
namespace {

struct NcDim { std::string name; long length; };
struct NcVar {
    std::string name;
    std::vector<int> dimids;
    int type;        // 1 byte, 2 char, 3 short, 4 int, 5 float, 6 double
    long long begin; // file offset of the data
    bool record;
};

struct NcFile {
    int fd = -1;
    long long size = 0;
    std::vector<NcDim> dims;
    std::vector<NcVar> vars;
    std::string error;

    ~NcFile() { if (fd >= 0) ::close(fd); }

    bool fail(const std::string &m) { error = m; return false; }

    bool read_at(long long off, void *dst, size_t n) {
        char *p = static_cast<char *>(dst);
        while (n > 0) {
            const ssize_t r = ::pread(fd, p, n, off);
            if (r < 0 && errno == EINTR) continue;
            if (r <= 0) return fail("unexpected end of file");
            p += r; off += r; n -= (size_t)r;
        }
        return true;
    }

    // --- header -------------------------------------------------------------------------------------
    std::vector<unsigned char> hdr;
    size_t pos = 0;
    bool need(size_t n) {
        while (pos + n > hdr.size()) {
            const size_t old = hdr.size();
            size_t grow = std::max<size_t>(old, 4096);
            if ((long long)(old + grow) > size) grow = (size_t)(size - (long long)old);
            if (grow == 0) return fail("truncated header");
            hdr.resize(old + grow);
            if (!read_at((long long)old, hdr.data() + old, grow)) return false;
        }
        return true;
    }
    bool u32(unsigned &v) {
        if (!need(4)) return false;
        v = ((unsigned)hdr[pos] << 24) | ((unsigned)hdr[pos + 1] << 16) | ((unsigned)hdr[pos + 2] << 8) | hdr[pos + 3];
        pos += 4;
        return true;
    }
    bool u64(unsigned long long &v) {
        unsigned hi, lo;
        if (!u32(hi) || !u32(lo)) return false;
        v = ((unsigned long long)hi << 32) | lo;
        return true;
    }
    bool name(std::string &s) {
        unsigned n;
        if (!u32(n)) return false;
        const size_t padded = (n + 3u) & ~3u;
        if (!need(padded)) return false;
        s.assign(reinterpret_cast<const char *>(hdr.data() + pos), n);
        pos += padded;
        return true;
    }
    static size_t type_size(int t) { return t == 1 || t == 2 ? 1 : t == 3 ? 2 : t == 4 || t == 5 ? 4 : t == 6 ? 8 : 0; }
    bool skip_attributes() {
        unsigned tag, n;
        if (!u32(tag) || !u32(n)) return false;
        if (tag == 0 && n == 0) return true;
        if (tag != 0x0C) return fail("malformed attribute list");
        for (unsigned i = 0; i < n; ++i) {
            std::string nm;
            unsigned type, count;
            if (!name(nm) || !u32(type) || !u32(count)) return false;
            const size_t ts = type_size((int)type);
            if (ts == 0) return fail("attribute '" + nm + "' has an unknown type");
            const size_t bytes = ((size_t)count * ts + 3u) & ~(size_t)3u;
            if (!need(bytes)) return false;
            pos += bytes;
        }
        return true;
    }

    bool open(const char *path) {
        fd = ::open(path, O_RDONLY);
        if (fd < 0) return fail(std::string("Could not open '") + path + "': " + std::strerror(errno));
        struct stat st;
        if (fstat(fd, &st) != 0) return fail("cannot stat the file");
        size = st.st_size;
        if (!need(4)) return false;
        if (hdr[0] != 'C' || hdr[1] != 'D' || hdr[2] != 'F') return fail("not a NetCDF classic file (no CDF magic)");
        const int version = hdr[3];
        if (version != 1 && version != 2)
            return fail("NetCDF format version " + std::to_string(version) + " is not the classic or 64-bit-offset format");
        pos = 4;
        unsigned numrecs, tag, n;
        if (!u32(numrecs)) return false;
        if (!u32(tag) || !u32(n)) return false;
        if (!(tag == 0 && n == 0)) {
            if (tag != 0x0A) return fail("malformed dimension list");
            for (unsigned i = 0; i < n; ++i) {
                NcDim d;
                unsigned len;
                if (!name(d.name) || !u32(len)) return false;
                d.length = len;  // 0 marks the record dimension
                dims.push_back(d);
            }
        }
        if (!skip_attributes()) return false;
        if (!u32(tag) || !u32(n)) return false;
        if (!(tag == 0 && n == 0)) {
            if (tag != 0x0B) return fail("malformed variable list");
            for (unsigned i = 0; i < n; ++i) {
                NcVar v;
                unsigned nd, type, vsize;
                if (!name(v.name) || !u32(nd)) return false;
                v.record = false;
                for (unsigned k = 0; k < nd; ++k) {
                    unsigned id;
                    if (!u32(id)) return false;
                    if (id >= dims.size()) return fail("variable '" + v.name + "' refers to an unknown dimension");
                    if (dims[id].length == 0) v.record = true;
                    v.dimids.push_back((int)id);
                }
                if (!skip_attributes() || !u32(type) || !u32(vsize)) return false;
                v.type = (int)type;
                if (version == 1) {
                    unsigned b;
                    if (!u32(b)) return false;
                    v.begin = b;
                } else {
                    unsigned long long b;
                    if (!u64(b)) return false;
                    v.begin = (long long)b;
                }
                vars.push_back(v);
            }
        }
        hdr.clear();
        hdr.shrink_to_fit();
        return true;
    }

    bool dimension(const char *nm, long &len) const {
        for (const NcDim &d : dims)
            if (d.name == nm) { len = d.length; return true; }
        return false;
    }
    const NcVar *variable(const char *nm) const {
        for (const NcVar &v : vars)
            if (v.name == nm) return &v;
        return nullptr;
    }
    long long elements(const NcVar &v) const {
        long long e = 1;
        for (int id : v.dimids) e *= dims[(size_t)id].length;
        return e;
    }

    // rows [row0, row0 + nrows) of a variable whose first dimension is the row index, as T (float or int)
    template <typename T>
    bool read_rows(const char *nm, int want_type, long long row0, long long nrows, long long row_len, T *dst) {
        const NcVar *v = variable(nm);
        if (!v) return fail(std::string("Cannot read array '") + nm + "': variable not found");
        if (v->record) return fail(std::string("variable '") + nm + "' uses the unlimited dimension, which is not supported");
        if (v->type != want_type) return fail(std::string("variable '") + nm + "' has an unexpected type");
        if (v->dimids.empty() || elements(*v) < (row0 + nrows) * row_len)
            return fail(std::string("Cannot read array '") + nm + "': index exceeds dimension bound");
        const size_t count = (size_t)(nrows * row_len);
        if (count == 0) return true;
        const size_t es = type_size(want_type);
        if (!read_at(v->begin + row0 * row_len * (long long)es, dst, count * es)) return false;
        if (es == 4) {
            unsigned *w = reinterpret_cast<unsigned *>(dst);
            for (size_t i = 0; i < count; ++i) w[i] = __builtin_bswap32(w[i]);
        }
        return true;
    }
};

struct Sequence {
    int original_seq_idx;  // index of this segment inside its utterance
    int length;
    long long begin;       // first row in inputs / targets
    std::string tag;
};

}  // namespace
}  // namespace cnt

struct cnt_dataset {
    cnt::NcFile file;
    cnt_dataset_desc desc;
    int input_size, output_size, is_classification;
    long total_timesteps;
    int min_len, max_len;
    std::vector<cnt::Sequence> sequences;
    std::mt19937 shuffle_gen;  // one generator for every shuffle of this data set, seeded by the first one
    bool shuffle_seeded = false;
};

namespace {

int dataset_error(cnt_dataset *d, const std::string &what) {
    cnt::set_error("%s", (what + (d && !d->file.error.empty() ? ": " + d->file.error : "")).c_str());
    return CNT_ERR_ARG;
}

}  // namespace

extern "C" {

int cnt_dataset_open(const char *nc_path, const cnt_dataset_desc *desc, cnt_dataset **out) {
    using namespace cnt;
    CNT_REQUIRE(nc_path && desc && out, "dataset_open: null argument");
    CNT_REQUIRE(desc->parallel_sequences >= 1, "dataset_open: parallel_sequences must be positive");
    // the reference's check (data_sets/DataSet.cpp:1322-1323)
    CNT_REQUIRE(desc->fraction > 0 && desc->fraction <= 1, "Invalid fraction");
    cnt_dataset *d = new (std::nothrow) cnt_dataset();
    CNT_REQUIRE(d != nullptr, "dataset_open: out of host memory");
    d->desc = *desc;
    auto bail = [&](const std::string &m) { const int s = dataset_error(d, m); delete d; return s; };
    if (!d->file.open(nc_path)) return bail("dataset_open");
    long max_tag, in_size, n_seq, n_steps = 0, labels = 0, out_size = 0;
    if (!d->file.dimension("maxSeqTagLength", max_tag)) return bail("Cannot get dimension 'maxSeqTagLength'");
    if (!d->file.dimension("inputPattSize", in_size)) return bail("Cannot get dimension 'inputPattSize'");
    d->is_classification = d->file.dimension("numLabels", labels) ? 1 : 0;
    if (d->is_classification) out_size = labels == 2 ? 1 : labels;
    else if (!d->file.dimension("targetPattSize", out_size)) return bail("Cannot get dimension 'targetPattSize'");
    if (!d->file.dimension("numSeqs", n_seq)) return bail("Cannot get dimension 'numSeqs'");
    d->file.dimension("numTimesteps", n_steps);
    // sizes a damaged header could claim
    constexpr long kMaxPattern = 1L << 20, kMaxTag = 1L << 16;
    if (in_size < 1 || in_size > kMaxPattern) return bail("dataset_open: dimension 'inputPattSize' out of range");
    if (out_size < 1 || out_size > kMaxPattern) return bail("dataset_open: target dimension out of range");
    if (max_tag < 1 || max_tag > kMaxTag) return bail("dataset_open: dimension 'maxSeqTagLength' out of range");
    if (n_seq < 1 || n_seq > (1L << 31) - 1) return bail("dataset_open: dimension 'numSeqs' out of range");
    if (n_steps < 0) return bail("dataset_open: dimension 'numTimesteps' out of range");
    d->input_size = (int)in_size;
    d->output_size = (int)out_size;

    int take = (int)((float)n_seq * desc->fraction);
    take = std::max(take, 1);
    if (take > n_seq) return bail("dataset_open: the file holds no sequence");
    std::vector<int> lengths((size_t)take);
    if (!d->file.read_rows<int>("seqLengths", 4, 0, take, 1, lengths.data())) return bail("dataset_open");
    std::vector<char> tags((size_t)take * (size_t)max_tag);
    if (!d->file.read_rows<char>("seqTags", 2, 0, take, max_tag, tags.data())) return bail("dataset_open");

    d->total_timesteps = 0;
    d->min_len = std::numeric_limits<int>::max();
    d->max_len = std::numeric_limits<int>::min();
    long long begin = 0;
    const int trunc = desc->truncate_seq;
    for (int i = 0; i < take; ++i) {
        int remaining = lengths[(size_t)i];
        if (remaining < 0) return bail("dataset_open: negative sequence length");
        d->total_timesteps += remaining;
        std::string tag(tags.data() + (size_t)i * (size_t)max_tag, (size_t)max_tag);
        tag = tag.c_str();  // cut at the first NUL, as the reference's std::string(buffer) does
        int k = 0;
        while (remaining > 0) {
            Sequence s;
            s.original_seq_idx = k;
            // a tail shorter than half a segment stays attached (data_sets/DataSet.cpp:1471-1477)
            s.length = (trunc > 0 && remaining > 1.5 * trunc) ? std::min(trunc, remaining) : remaining;
            s.begin = begin;
            s.tag = tag;
            d->sequences.push_back(s);
            d->min_len = std::min(d->min_len, s.length);
            d->max_len = std::max(d->max_len, s.length);
            begin += s.length;
            remaining -= s.length;
            ++k;
        }
    }
    if (n_steps > 0 && begin > n_steps) return bail("dataset_open: seqLengths add up to more than numTimesteps");
    if (d->sequences.empty()) return bail("dataset_open: the file holds no time step");
    // the reference uses std::sort, which leaves the order of equal lengths unspecified; here it is stable
    if (desc->training_mode)
        std::stable_sort(d->sequences.begin(), d->sequences.end(),
                         [](const Sequence &a, const Sequence &b) { return a.length < b.length; });
    *out = d;
    return CNT_OK;
}

// DataSet::_shuffleSequences / _shuffleFractions (data_sets/DataSet.cpp:491-514), run by the reference at the start of
// every epoch (:1026-1031): first the sequences are shuffled, then the groups of parallel_sequences consecutive
// sequences, whose concatenation becomes the new order (a last, shorter group may land in the middle, and the
// fractions after it then straddle the old groups, as in the reference).  The shuffle is the one std::random_shuffle
// of libstdc++ runs -- element i changes places with a uniformly drawn element of 0..i -- on one Mersenne twister per
// data set that the first call seeds (the reference seeds one per process from --random_seed and draws through
// boost::uniform_int, so the permutations themselves are not the reference's).
int cnt_dataset_shuffle(cnt_dataset *d, int shuffle_sequences, int shuffle_fractions, unsigned seed) {
    using namespace cnt;
    CNT_REQUIRE(d, "dataset_shuffle: null handle");
    if (!d->shuffle_seeded) {
        d->shuffle_gen.seed(seed);
        d->shuffle_seeded = true;
    }
    auto below = [&](size_t n) {  // uniform in 0 .. n-1, without modulo bias
        const unsigned long long span = 0x100000000ull, lim = span - span % n;
        unsigned long long r;
        do r = d->shuffle_gen(); while (r >= lim);
        return (size_t)(r % n);
    };
    auto shuffle = [&](auto &v) {
        for (size_t i = 1; i < v.size(); ++i) {
            const size_t j = below(i + 1);
            if (i != j) std::swap(v[i], v[j]);
        }
    };
    if (shuffle_sequences) shuffle(d->sequences);
    if (shuffle_fractions) {
        const size_t S = (size_t)d->desc.parallel_sequences;
        std::vector<std::vector<Sequence>> groups;
        for (size_t i = 0; i < d->sequences.size(); ++i) {
            if (i % S == 0) groups.emplace_back();
            groups.back().push_back(d->sequences[i]);
        }
        shuffle(groups);
        d->sequences.clear();
        for (const auto &g : groups)
            for (const auto &q : g) d->sequences.push_back(q);
    }
    return CNT_OK;
}

int cnt_dataset_close(cnt_dataset *d) {
    delete d;
    return CNT_OK;
}

int cnt_dataset_info(cnt_dataset *d, int *num_sequences, int *input_size, int *output_size, int *is_classification,
                     long *total_timesteps, int *min_len, int *max_len) {
    using namespace cnt;
    CNT_REQUIRE(d, "dataset_info: null handle");
    if (num_sequences) *num_sequences = (int)d->sequences.size();
    if (input_size) *input_size = d->input_size;
    if (output_size) *output_size = d->output_size;
    if (is_classification) *is_classification = d->is_classification;
    if (total_timesteps) *total_timesteps = d->total_timesteps;
    if (min_len) *min_len = d->min_len;
    if (max_len) *max_len = d->max_len;
    return CNT_OK;
}

int cnt_dataset_sequence(cnt_dataset *d, int index, int *length, int *original_seq_idx, char *tag, int tag_cap) {
    using namespace cnt;
    CNT_REQUIRE(d && index >= 0 && index < (int)d->sequences.size(), "dataset_sequence: index out of range");
    const Sequence &s = d->sequences[(size_t)index];
    if (length) *length = s.length;
    if (original_seq_idx) *original_seq_idx = s.original_seq_idx;
    if (tag && tag_cap > 0) {
        std::strncpy(tag, s.tag.c_str(), (size_t)tag_cap - 1);
        tag[tag_cap - 1] = '\0';
    }
    return CNT_OK;
}

int cnt_dataset_fraction_shape(cnt_dataset *d, int first_seq, int *num_seqs, int *max_len, int *min_len,
                               int *total_length) {
    using namespace cnt;
    CNT_REQUIRE(d && first_seq >= 0 && first_seq < (int)d->sequences.size(), "dataset_fraction: first sequence out of range");
    int n = 0, mx = std::numeric_limits<int>::min(), mn = std::numeric_limits<int>::max(), total = 0;
    for (int i = first_seq; i < first_seq + d->desc.parallel_sequences && i < (int)d->sequences.size(); ++i) {
        const int len = d->sequences[(size_t)i].length;
        mx = std::max(mx, len); mn = std::min(mn, len); total += len; ++n;
    }
    if (num_seqs) *num_seqs = n;
    if (max_len) *max_len = mx;
    if (min_len) *min_len = mn;
    if (total_length) *total_length = total;
    return CNT_OK;
}

int cnt_dataset_fraction_fill(cnt_dataset *d, int first_seq, char *patTypes, float *inputs, float *targets,
                              int *target_classes) {
    using namespace cnt;
    int n, T;
    CNT_TRY(cnt_dataset_fraction_shape(d, first_seq, &n, &T, nullptr, nullptr));
    CNT_REQUIRE(patTypes && inputs, "dataset_fraction: null buffer");
    CNT_REQUIRE(d->is_classification ? target_classes != nullptr : targets != nullptr,
                "dataset_fraction: the target buffer of this data set's kind is missing");
    const int S = d->desc.parallel_sequences, P = d->input_size, Q = d->output_size;
    const size_t slots = (size_t)T * S;
    std::memset(patTypes, 0, slots);
    std::fill(inputs, inputs + slots * P, 0.0f);
    if (d->is_classification) std::fill(target_classes, target_classes + slots, -1);
    else std::fill(targets, targets + slots * Q, 0.0f);
    std::vector<float> rows;
    std::vector<int> classes;
    for (int i = 0; i < n; ++i) {
        const Sequence &s = d->sequences[(size_t)(first_seq + i)];
        rows.resize((size_t)s.length * P);
        if (!d->file.read_rows<float>("inputs", 5, s.begin, s.length, P, rows.data())) return dataset_error(d, "dataset_fraction");
        for (int t = 0; t < s.length; ++t)
            std::memcpy(inputs + ((size_t)t * S + i) * P, rows.data() + (size_t)t * P, sizeof(float) * P);
        if (d->is_classification) {
            classes.resize((size_t)s.length);
            if (!d->file.read_rows<int>("targetClasses", 4, s.begin, s.length, 1, classes.data()))
                return dataset_error(d, "dataset_fraction");
            for (int t = 0; t < s.length; ++t) target_classes[(size_t)t * S + i] = classes[(size_t)t];
        } else {
            rows.resize((size_t)s.length * Q);
            if (!d->file.read_rows<float>("targetPatterns", 5, s.begin, s.length, Q, rows.data()))
                return dataset_error(d, "dataset_fraction");
            for (int t = 0; t < s.length; ++t)
                std::memcpy(targets + ((size_t)t * S + i) * Q, rows.data() + (size_t)t * Q, sizeof(float) * Q);
        }
        for (int t = 0; t < s.length; ++t)
            patTypes[(size_t)t * S + i] = t == 0 ? 1 : (t == s.length - 1 ? 3 : 2);  // FIRST, LAST, NORMAL
    }
    return CNT_OK;
}

}  // extern "C"
