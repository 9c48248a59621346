// Runs the CPU-only parts of the host layer (number theory, BLAKE2b, table construction, record save / load) under
// AddressSanitizer + UndefinedBehaviorSanitizer, against the host-memory mock of the device ABI (mock_device.cpp).
// Ends with a bounded, seeded loop that feeds damaged and random records to every load() entry: a parser may refuse
// a record (any std::exception), it may not crash or touch memory it does not own.  Exit code 0 = clean.
#include <cstdio>
#include <cstring>
#include <random>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "cahel.h"

using namespace cahel;

#define REQUIRE(cond)                                                        \
    do {                                                                     \
        if (!(cond)) {                                                       \
            std::fprintf(stderr, "REQUIRE failed: %s (line %d)\n", #cond, __LINE__); \
            return 1;                                                        \
        }                                                                    \
    } while (0)

template <typename T>
static std::string saved(const T &obj) {
    std::ostringstream os(std::ios::binary);
    obj.save(os);
    return os.str();
}

template <typename F>
static bool refuses(F &&f) {
    try {
        f();
    } catch (const std::exception &) {
        return true;
    }
    return false;
}

int main(int argc, char **argv) {
    const long rounds = argc > 1 ? std::atol(argv[1]) : 20000;

    // ---- number theory known answers (cahel-main/unittest/util/numth.cu, the reference's own vectors) ----
    uint64_t root = 0;
    REQUIRE(try_minimal_primitive_root(2, 11, root) && root == 10);
    REQUIRE(try_minimal_primitive_root(4, 29, root) && root == 12);
    REQUIRE(try_minimal_primitive_root(8, 1234565441ull, root) && root == 249725733ull);
    const auto primes = get_primes(8192, 44, 3);
    REQUIRE(primes.size() == 3 && primes[0] == 0xfffffffc001ull && primes[1] == 0xffffff6c001ull &&
            primes[2] == 0xfffffebc001ull);
    const auto digits = naf(-7);  // -8 + 1
    REQUIRE(!digits.empty());
    long sum = 0;
    for (int d : digits) sum += d;
    REQUIRE(sum == -7);
    // RFC 7693 appendix A: BLAKE2b-512("abc") starts ba 80 a5 3f
    unsigned char digest[64];
    blake2b(digest, 64, "abc", 3);
    REQUIRE(digest[0] == 0xba && digest[1] == 0x80 && digest[2] == 0xa5 && digest[3] == 0x3f && digest[63] == 0x23);

    // ---- context: every table of every level is built on the host and handed to the (mock) device ----
    const std::size_t n = 1024;
    EncryptionParameters parms(scheme_type::ckks);
    parms.set_poly_modulus_degree(n);
    parms.set_coeff_modulus(CoeffModulus::Create(n, {40, 30, 30, 30, 30, 30, 40, 40}));
    parms.set_special_modulus_size(2);   // six data limbs, three digits of two
    parms.set_galois_elts(get_elts_from_steps({1, -1, 0, 5}, n));
    CAHELGPUContext context(parms, true, sec_level_type::none);
    REQUIRE(context.size_q() == 6 && context.size_p() == 2);
    REQUIRE(context.limbs_at(1) == context.size_q());
    REQUIRE(context.parms_id_at(0) != context.parms_id_at(1));

    // ---- parameters record ----
    const std::string prec = saved(parms);
    {
        EncryptionParameters back;
        std::istringstream is(prec, std::ios::binary);
        back.load(is);
        REQUIRE(back.poly_modulus_degree() == n && back.coeff_modulus().size() == parms.coeff_modulus().size());
        REQUIRE(back.coeff_modulus()[3].value() == parms.coeff_modulus()[3].value());
    }

    // ---- plaintext and ciphertext records over the mock's host memory ----
    CAHELGPUPlaintext plain(context);
    plain.resize(context.limbs_at(1), n);
    plain.chain_index() = 1;
    plain.parms_id() = context.parms_id_at(1);
    plain.scale() = 1099511627776.0;
    for (std::size_t i = 0; i < context.limbs_at(1) * n; i++) plain.data()[i] = i * 2654435761u;
    CAHELGPUCiphertext cipher(context);
    cipher.resize(context, 2, 3);
    cipher.scale() = 1048576.0;
    for (std::size_t i = 0; i < 3 * context.limbs_at(2) * n; i++) cipher.data()[i] = i * 40503u + 7;
    const std::string ptrec = saved(plain), ctrec = saved(cipher);
    {
        CAHELGPUPlaintext back(context);
        std::istringstream is(ptrec, std::ios::binary);
        back.load(context, is);
        REQUIRE(back.chain_index() == 1 && back.scale() == plain.scale());
        REQUIRE(std::memcmp(back.data(), plain.data(), context.limbs_at(1) * n * 8) == 0);
        CAHELGPUCiphertext cback(context);
        std::istringstream cs(ctrec, std::ios::binary);
        cback.load(context, cs);
        REQUIRE(cback.size() == 3 && cback.chain_index() == 2 && cback.coeff_modulus_size() == context.limbs_at(2));
        REQUIRE(std::memcmp(cback.data(), cipher.data(), 3 * context.limbs_at(2) * n * 8) == 0);
        // copy / shrink / grow of a ciphertext keep the leading words and stay inside their block
        CAHELGPUCiphertext copy = cback;
        copy.resize(2, copy.coeff_modulus_size(), n);
        CAHELGPUCiphertext copy2 = copy;
        REQUIRE(copy2.size() == 2 && std::memcmp(copy2.data(), cipher.data(), 2 * context.limbs_at(2) * n * 8) == 0);
        copy.resize(3, copy.coeff_modulus_size(), n);
        REQUIRE(std::memcmp(copy.data(), cipher.data(), 2 * context.limbs_at(2) * n * 8) == 0);
    }
    // ---- device blocks: slices, shared owners, and a key switch that is deferred past its key's lifetime ----
    {
        auto parent = std::make_shared<DeviceBuffer>(4 * n);
        for (std::size_t i = 0; i < 4 * n; i++) parent->get()[i] = i;
        DeviceBuffer s1 = DeviceBuffer::slice(parent, n, n), s2 = DeviceBuffer::slice(parent, 3 * n, n);
        parent.reset();                       // the slices keep the block
        REQUIRE(s1.get()[0] == n && s2.get()[n - 1] == 4 * n - 1);
        REQUIRE(refuses([&] { DeviceBuffer::slice(s1.owner(), 4 * n, 1); }));
        DeviceBuffer own(n);
        for (std::size_t i = 0; i < n; i++) own.get()[i] = 7 * i;
        s1 = own;                             // copy-assign into a slice of the same size: the words land in the parent's block
        REQUIRE(s1.get()[5] == 35 && s1.owner());
        DeviceBuffer big(2 * n);
        for (std::size_t i = 0; i < 2 * n; i++) big.get()[i] = i + 1;
        s1.assign(big, 2 * n);                // larger than the slice: it takes a block of its own
        REQUIRE(s1.words() == 2 * n && !s1.owner() && s1.get()[2 * n - 1] == 2 * n);
        { DeviceBuffer last = std::move(s2); }   // the last slice to go frees the parent's block
        // a ciphertext whose block is a slice: growing it past the slice moves it to a block of its own
        auto batch = std::make_shared<DeviceBuffer>(4 * context.limbs_at(2) * n);
        for (std::size_t i = 0; i < batch->words(); i++) batch->get()[i] = 3 * i;
        CAHELGPUCiphertext part(context);
        part.adopt(DeviceBuffer::slice(batch, 2 * context.limbs_at(2) * n, 2 * context.limbs_at(2) * n));
        part.size_ = 2;
        part.coeff_modulus_size_ = context.limbs_at(2);
        part.poly_modulus_degree_ = n;
        batch.reset();
        const uint64_t first = part.data()[0];
        part.resize(3, part.coeff_modulus_size(), n);
        REQUIRE(part.data()[0] == first && !part.data_.owner());
        // make_shared keeps the words in place; owners outlive the object that made them
        DeviceBuffer key(2 * context.size_qp() * n);
        for (std::size_t i = 0; i < key.words(); i++) key.get()[i] = i ^ 0x55;
        const uint64_t *where = key.get();
        key.make_shared();
        REQUIRE(key.get() == where && key.owner() && key.owner().use_count() == 1);
        // a relinearisation deferred on `three` (as relinearize_inplace leaves it) while its key object goes away
        const std::size_t L2 = context.limbs_at(2);
        CAHELGPUCiphertext three(context);
        three.resize(context, 2, 3);
        for (std::size_t i = 0; i < 3 * L2 * n; i++) three.data()[i] = i;
        auto pending = std::make_shared<PendingKeySwitch>();
        pending->handle = context.handle();
        pending->limbs = (uint32_t)L2;
        std::vector<DeviceBuffer> digits((L2 + context.size_p() - 1) / context.size_p());
        for (auto &d : digits) {
            d.allocate(2 * context.size_qp() * n);
            std::memset(d.get(), 1, d.words() * 8);
            d.make_shared();
            pending->key_ptrs.push_back(d.get());
            pending->key_owners.push_back(d.owner());
        }
        three.size_ = 2;
        three.pending_ = pending;
        pending.reset();
        digits.clear();                       // the key is gone; the owners in the pending switch keep its blocks
        DeviceBuffer::trim_pool();
        REQUIRE(three.has_pending_key_switch() && three.size() == 2);
        CAHELGPUCiphertext after = three;     // a copy runs the switch on the source first
        REQUIRE(!three.has_pending_key_switch() && !after.has_pending_key_switch());
        REQUIRE(three.data()[0] == 1 && after.data()[1] == 2 && after.size() == 2);   // the mock adds one to (c0, c1)
        three.pending_ = std::make_shared<PendingKeySwitch>();   // overwritten as a whole: nothing runs
        three.adopt(DeviceBuffer(2 * L2 * n));
        REQUIRE(!three.has_pending_key_switch());
    }

    // a record of another level, a truncated one and one with a wrong degree are refused
    REQUIRE(refuses([&] {
        std::string bad = ctrec.substr(0, ctrec.size() / 2);
        std::istringstream is(bad, std::ios::binary);
        CAHELGPUCiphertext c(context);
        c.load(context, is);
    }));

    // ---- bounded fuzz: damaged copies of the valid records and pure noise into every loader ----
    std::mt19937_64 rng(20250117);
    long refused = 0, accepted = 0;
    const std::string *seeds[3] = {&prec, &ptrec, &ctrec};
    for (long it = 0; it < rounds; it++) {
        std::string rec;
        const int kind = (int)(rng() % 4);
        if (kind == 3) {
            rec.resize(rng() % 200);
            for (auto &ch : rec) ch = (char)rng();
        } else {
            rec = *seeds[kind];
            // headers sit in the first bytes: damage mostly there, sometimes anywhere, sometimes truncate
            const int hits = 1 + (int)(rng() % 4);
            for (int h = 0; h < hits; h++) {
                const std::size_t span = (rng() & 3) ? std::min<std::size_t>(rec.size(), 96) : rec.size();
                rec[rng() % span] = (char)rng();
            }
            if ((rng() & 7) == 0) rec.resize(rng() % rec.size());
        }
        const int target = (int)(rng() % 6);
        const bool bad = refuses([&] {
            std::istringstream is(rec, std::ios::binary);
            switch (target) {
                case 0: { EncryptionParameters p; p.load(is); break; }
                case 1: { CAHELGPUPlaintext p(context); p.load(context, is); break; }
                case 2: { CAHELGPUCiphertext c(context); c.load(context, is); break; }
                case 3: { CAHELGPUPublicKey k(context); k.load(context, is); break; }
                case 4: { CAHELGPURelinKey k; k.load(context, is); break; }
                default: { CAHELGPUGaloisKey k(context); k.load(context, is); break; }
            }
        });
        (bad ? refused : accepted)++;
    }
    std::printf("host sanitize driver ok: %ld records refused, %ld accepted\n", refused, accepted);
    return 0;
}
