// Wire format of plaintexts, ciphertexts and keys: the byte layout that the reference's save()/load() members
// produce (cahel-main/include/plaintext.h:109-200, include/ciphertext.h:174-290, include/secretkey.h:53-59,
// 212-256, 354-398), so that files written by either side can be read by the other.  Everything is little-endian
// and unpadded:
//
//   parameters  scheme u8 | N u64 | count u64 | moduli[count] u64 | plain modulus u64 (include/util/
//               encryptionparams.h:381-474, src/modulus.cu:134-178)
//   plaintext   parms_id[32] | limbs u64 | chain u64 | N u64 | scale f64 | words u64 | data[words] u64
//   ciphertext  parms_id[32] | ntt u8 | chain u64 | size u64 | N u64 | limbs u64 | scale f64 | words u64 |
//               data[words] u64 | seed[64]
//   public key  one ciphertext record (size 2, key level)
//   relin key   parms_id[32] | generated u8 | count u64 | count public-key records (one per digit)
//   Galois key  parms_id[32] | generated u8 | count u64 | count relin-key records (one per Galois element)
//
// The reference loads whatever the header says.  Here load() also checks the header against the context (degree,
// chain index, limb count of that level, parms_id, word count) and throws std::invalid_argument on a mismatch:
// these objects index device tables by chain index, so a record of another parameter set must not get in.  Stream
// failures give std::runtime_error("I/O error") as in the reference.
#include <cstring>
#include <istream>
#include <ostream>

#include "cahel.h"

using namespace cahel;

namespace {

// restores the stream's exception mask on scope exit and maps stream failures to the reference's error
class StreamGuard {
public:
    explicit StreamGuard(std::ios &stream) : stream_(stream), mask_(stream.exceptions()) {
        stream_.exceptions(std::ios_base::badbit | std::ios_base::failbit);
    }
    ~StreamGuard() {
        try {
            stream_.exceptions(mask_);
        } catch (...) {
            // restoring a mask that covers a bit already set throws: the caller sees the first error instead
        }
    }

private:
    std::ios &stream_;
    std::ios_base::iostate mask_;
};

template <typename F>
void io_section(std::ios &stream, F &&body) {
    StreamGuard guard(stream);
    try {
        body();
    } catch (const std::ios_base::failure &) {
        throw std::runtime_error("I/O error");
    }
}

template <typename T>
void put(std::ostream &s, const T &v) {
    s.write(reinterpret_cast<const char *>(&v), sizeof(T));
}

template <typename T>
T get(std::istream &s) {
    T v{};
    s.read(reinterpret_cast<char *>(&v), sizeof(T));
    return v;
}

void put_device_words(std::ostream &s, const uint64_t *dev, std::size_t words) {
    put<uint64_t>(s, words);
    std::vector<uint64_t> host(words);
    if (words)
        check_status(he_memcpy_d2h(host.data(), dev, words * sizeof(uint64_t), current_stream()), "download");
    s.write(reinterpret_cast<const char *>(host.data()), (std::streamsize)(words * sizeof(uint64_t)));
}

void get_device_words(std::istream &s, uint64_t *dev, std::size_t words) {
    if (get<uint64_t>(s) != words) throw std::invalid_argument("data size does not match the header");
    std::vector<uint64_t> host(words);
    s.read(reinterpret_cast<char *>(host.data()), (std::streamsize)(words * sizeof(uint64_t)));
    if (words) check_status(he_memcpy_h2d(dev, host.data(), words * sizeof(uint64_t), current_stream()), "upload");
}

// header fields against the context: every object of the chain has the context's degree and its level's limbs
void check_header(const CAHELGPUContext &context, const parms_id_type &id, uint64_t chain, uint64_t degree,
                  uint64_t limbs) {
    if (degree != context.poly_degree()) throw std::invalid_argument("poly_modulus_degree does not match the context");
    if (chain >= context.chain_size()) throw std::invalid_argument("chain index out of range");
    if (limbs != context.limbs_at((std::size_t)chain)) throw std::invalid_argument("coeff_modulus_size does not match the chain index");
    if (id != context.parms_id_at((std::size_t)chain)) throw std::invalid_argument("parms_id does not match the context");
}

}  // namespace

// ---------------------------------------------------------------------------------------------------
// parameters
// ---------------------------------------------------------------------------------------------------
void EncryptionParameters::save(std::ostream &stream) const {
    io_section(stream, [&] {
        put<uint8_t>(stream, (uint8_t)scheme_);
        put<uint64_t>(stream, poly_modulus_degree_);
        put<uint64_t>(stream, coeff_modulus_.size());
        for (const auto &m : coeff_modulus_) put<uint64_t>(stream, m.value());
        put<uint64_t>(stream, 0);  // plain modulus: BFV / BGV only
    });
}

void EncryptionParameters::load(std::istream &stream) {
    io_section(stream, [&] {
        const uint8_t scheme = get<uint8_t>(stream);
        if (scheme > (uint8_t)scheme_type::ckks) throw std::invalid_argument("unsupported scheme");
        EncryptionParameters fresh((scheme_type)scheme);
        const uint64_t degree = get<uint64_t>(stream), count = get<uint64_t>(stream);
        if (degree > 131072) throw std::logic_error("poly_modulus_degree is invalid");  // CAHEL_POLY_MOD_DEGREE_MAX
        if (count > 64) throw std::logic_error("coeff_modulus is invalid");
        std::vector<Modulus> moduli;
        for (uint64_t i = 0; i < count; i++) moduli.emplace_back(get<uint64_t>(stream));
        if (get<uint64_t>(stream) != 0 && (scheme_type)scheme == scheme_type::ckks)
            throw std::logic_error("plain_modulus is not supported for this scheme");
        fresh.set_poly_modulus_degree((std::size_t)degree);
        fresh.set_coeff_modulus(moduli);
        *this = std::move(fresh);
    });
}

// ---------------------------------------------------------------------------------------------------
// plaintext
// ---------------------------------------------------------------------------------------------------
void CAHELGPUPlaintext::save(std::ostream &stream) const {
    io_section(stream, [&] {
        put(stream, parms_id_);
        put<uint64_t>(stream, coeff_modulus_size_);
        put<uint64_t>(stream, chain_index_);
        put<uint64_t>(stream, poly_modulus_degree_);
        put<double>(stream, scale_);
        put_device_words(stream, data(), coeff_modulus_size_ * poly_modulus_degree_);
    });
}

void CAHELGPUPlaintext::load(const CAHELGPUContext &context, std::istream &stream) {
    CAHELGPUPlaintext fresh(context);
    io_section(stream, [&] {
        const auto id = get<parms_id_type>(stream);
        const uint64_t limbs = get<uint64_t>(stream), chain = get<uint64_t>(stream), degree = get<uint64_t>(stream);
        const double scale = get<double>(stream);
        check_header(context, id, chain, degree, limbs);
        fresh.resize((std::size_t)limbs, (std::size_t)degree);
        fresh.parms_id_ = id;
        fresh.chain_index_ = (std::size_t)chain;
        fresh.scale_ = scale;
        get_device_words(stream, fresh.data(), (std::size_t)(limbs * degree));
    });
    *this = std::move(fresh);
}

// ---------------------------------------------------------------------------------------------------
// ciphertext
// ---------------------------------------------------------------------------------------------------
void CAHELGPUCiphertext::save(std::ostream &stream) const {
    io_section(stream, [&] {
        put(stream, parms_id_);
        put<uint8_t>(stream, is_ntt_form_ ? 1 : 0);
        put<uint64_t>(stream, chain_index_);
        put<uint64_t>(stream, size_);
        put<uint64_t>(stream, poly_modulus_degree_);
        put<uint64_t>(stream, coeff_modulus_size_);
        put<double>(stream, scale_);
        put_device_words(stream, data(), size_ * coeff_modulus_size_ * poly_modulus_degree_);
        stream.write(reinterpret_cast<const char *>(prng_seed_.data()), (std::streamsize)prng_seed_.size());
    });
}

void CAHELGPUCiphertext::load(const CAHELGPUContext &context, std::istream &stream) {
    CAHELGPUCiphertext fresh(context);
    io_section(stream, [&] {
        const auto id = get<parms_id_type>(stream);
        const bool ntt = get<uint8_t>(stream) != 0;
        const uint64_t chain = get<uint64_t>(stream), size = get<uint64_t>(stream), degree = get<uint64_t>(stream),
                       limbs = get<uint64_t>(stream);
        const double scale = get<double>(stream);
        check_header(context, id, chain, degree, limbs);
        if (size < 2 || size > 3) throw std::invalid_argument("ciphertext size must be 2 or 3");
        fresh.resize((std::size_t)size, (std::size_t)limbs, (std::size_t)degree);
        fresh.parms_id_ = id;
        fresh.is_ntt_form_ = ntt;
        fresh.chain_index_ = (std::size_t)chain;
        fresh.scale_ = scale;
        get_device_words(stream, fresh.data(), (std::size_t)(size * limbs * degree));
        stream.read(reinterpret_cast<char *>(fresh.prng_seed_.data()), (std::streamsize)fresh.prng_seed_.size());
    });
    *this = std::move(fresh);
}

// ---------------------------------------------------------------------------------------------------
// keys
// ---------------------------------------------------------------------------------------------------
void CAHELGPUPublicKey::save(std::ostream &stream) const { pk_.save(stream); }

void CAHELGPUPublicKey::load(const CAHELGPUContext &context, std::istream &stream) {
    CAHELGPUCiphertext fresh(context);
    fresh.load(context, stream);
    if (fresh.chain_index() != 0 || fresh.size() != 2) throw std::invalid_argument("not a key-level pair");
    pk_ = std::move(fresh);
    gen_flag_ = true;
}

void CAHELGPURelinKey::save(std::ostream &stream) const {
    io_section(stream, [&] {
        put(stream, parms_id_);
        put<uint8_t>(stream, gen_flag_ ? 1 : 0);
        put<uint64_t>(stream, pk_num_);
    });
    for (std::size_t i = 0; i < pk_num_; i++) public_keys_[i].save(stream);
}

void CAHELGPURelinKey::load(const CAHELGPUContext &context, std::istream &stream) {
    parms_id_type id{};
    bool generated = false;
    uint64_t count = 0;
    io_section(stream, [&] {
        id = get<parms_id_type>(stream);
        generated = get<uint8_t>(stream) != 0;
        count = get<uint64_t>(stream);
    });
    if (id != context.key_parms_id()) throw std::invalid_argument("parms_id does not match the context");
    const std::size_t dnum = context.size_p() ? context.size_q() / context.size_p() : 0;
    if (count != dnum) throw std::invalid_argument("key count does not match the number of digits");
    std::vector<CAHELGPUPublicKey> fresh((std::size_t)count);
    for (auto &pk : fresh) {
        pk.load(context, stream);
        pk.pk_.data_.make_shared();   // as generate_one_kswitch_key leaves them
    }
    public_keys_ = std::move(fresh);
    pk_num_ = (std::size_t)count;
    gen_flag_ = generated;
    parms_id_ = id;
}

void CAHELGPUGaloisKey::save(std::ostream &stream) const {
    io_section(stream, [&] {
        put(stream, parms_id_);
        put<uint8_t>(stream, gen_flag_ ? 1 : 0);
        put<uint64_t>(stream, relin_key_num_);
    });
    for (std::size_t i = 0; i < relin_key_num_; i++) relin_keys_[i].save(stream);
}

void CAHELGPUGaloisKey::load(const CAHELGPUContext &context, std::istream &stream) {
    parms_id_type id{};
    bool generated = false;
    uint64_t count = 0;
    io_section(stream, [&] {
        id = get<parms_id_type>(stream);
        generated = get<uint8_t>(stream) != 0;
        count = get<uint64_t>(stream);
    });
    if (id != context.key_parms_id()) throw std::invalid_argument("parms_id does not match the context");
    // key i belongs to Galois element i of the context (src/secretkey.cu: create_galois_keys walks galois_elts)
    if (count != context.galois_elts().size()) throw std::invalid_argument("key count does not match the Galois elements");
    std::vector<CAHELGPURelinKey> fresh((std::size_t)count);
    for (auto &rk : fresh) rk.load(context, stream);
    relin_keys_ = std::move(fresh);
    relin_key_num_ = (std::size_t)count;
    gen_flag_ = generated;
    parms_id_ = id;
}
