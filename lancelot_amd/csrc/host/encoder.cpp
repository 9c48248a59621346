// CKKS encoder: slots <-> plaintext polynomial through the canonical embedding restricted to the orbit
// 5^j mod 2N (cahel-main/src/ckks.cu:34-209 encode, :292-465 decode; transform of src/fft.cu; rounding and
// residues of src/rns_base.cu:121-156; CRT composition of src/rns_base.cu:325-459).
//
// Everything runs on the GPU (he_ckks_encode / he_ckks_decode: special FFT of HEAAN's fftSpecial / fftSpecialInv
// butterfly network in FP64, rounding, residues, CRT composition, NTTs); the host moves the slot values in and
// out and keeps the reference's argument checks.  Decoded values agree with the reference up to FP64 operation
// order (bounded by the 2^-20 acceptance tolerance), not bit for bit.
#include <cmath>
#include <cstring>

#include "cahel.h"

using namespace cahel;

namespace {

// Page-locked staging for the values of an encoding, one buffer per host thread (the lanes of the host layer encode
// from several threads), grown on demand and kept until the thread ends.  The values are copied into it and uploaded
// without waiting; every encoding ends with a blocking download (its largest coefficient), after which the buffer is
// free for the thread's next call.
struct PinnedStage {
    void *ptr = nullptr;
    std::size_t bytes = 0;
    PinnedStage() = default;
    PinnedStage(const PinnedStage &) = delete;
    PinnedStage &operator=(const PinnedStage &) = delete;
    ~PinnedStage() {
        if (ptr) (void)he_host_free(ptr);   // (worker threads of a pool come and go: no buffer is left behind)
    }
    double *ensure(std::size_t want) {
        if (want > bytes) {
            void *old = ptr;
            ptr = nullptr;
            bytes = 0;
            if (old) check_status(he_host_free(old), "he_host_free");
            check_status(he_host_malloc(&ptr, want), "he_host_malloc");
            bytes = want;
        }
        return static_cast<double *>(ptr);
    }
};

double *pinned_stage(std::size_t bytes) {
    thread_local PinnedStage stage;
    return stage.ensure(bytes);
}

}  // namespace

CAHELGPUCKKSEncoder::CAHELGPUCKKSEncoder(const CAHELGPUContext &context) {
    if (context.scheme() != scheme_type::ckks) throw std::invalid_argument("unsupported scheme");
    slots_ = context.poly_degree() >> 1;
    first_chain_index_ = context.get_first_index();
}

std::size_t CAHELGPUCKKSEncoder::message_slots(std::size_t count) {
    if (sparse_slots_ == 0) {
        // the first message fixes the slot count for the lifetime of the encoder (src/ckks.cu:131-142)
        std::size_t s = 1;
        while (s < count) s <<= 1;
        sparse_slots_ = s;
    } else if (count > sparse_slots_) {
        throw std::invalid_argument("values_size exceeds previous message length");
    }
    if (sparse_slots_ < 2) throw std::invalid_argument("single value encoding is not available");
    return sparse_slots_;
}

std::vector<CAHELGPUCiphertext> CAHELGPUCKKSEncoder::encode_encrypt_many(const CAHELGPUContext &context,
                                                                         const CAHELGPUPublicKey &pk, const double *values,
                                                                         std::size_t items, std::size_t count,
                                                                         std::size_t value_stride, double scale) {
    if (items == 0) return {};
    if (items > 8192) throw std::invalid_argument("too many messages");
    if (!pk.gen_flag_) throw std::logic_error("public key has not been generated");
    if (count > slots_ || value_stride < count) throw std::invalid_argument("values_size is too large");
    const std::size_t chain = first_chain_index_;
    if (chain == 0 || context.size_p() == 0) throw std::logic_error("batched encryption needs a data level and special primes");
    const int total_bits = context.total_coeff_modulus_bit_count(chain);
    if (scale <= 0 || (static_cast<int>(std::log2(scale)) + 1 >= total_bits))
        throw std::invalid_argument("scale out of bounds");
    const std::size_t ss = message_slots(count);
    const std::size_t n = context.poly_degree();
    const uint32_t L = (uint32_t)context.limbs_at(chain);
    he_context *h = context.handle();
    he_stream st = context.stream();

    // values -> device, packed
    DeviceBuffer staging(items * count);
    double *d_values = reinterpret_cast<double *>(staging.get());
    if (count) {
        if (value_stride == count) {
            check_status(he_memcpy_h2d(d_values, values, items * count * sizeof(double), st), "upload");
        } else {
            for (std::size_t k = 0; k < items; k++)
                check_status(he_memcpy_h2d(d_values + k * count, values + k * value_stride, count * sizeof(double), st), "upload");
        }
    }
    // plaintexts straight into polynomial 0 of the ciphertexts
    const std::size_t words = 2 * (std::size_t)L * n;
    DeviceBuffer batch(items * words), ws(he_ckks_encode_batch_workspace_words(h, (uint32_t)items));
    check_status(he_ckks_encode_batch(h, d_values, nullptr, (uint32_t)count, (uint32_t)ss, scale, L, (uint32_t)items, count,
                                      batch.get(), 2 * L, ws.get(), st),
                 "he_ckks_encode_batch");
    std::vector<double> maxima(items);
    check_status(he_memcpy_d2h(maxima.data(), ws.get(), items * sizeof(double), st), "download");
    for (double max_coeff : maxima) {
        const int max_coeff_bit_count = static_cast<int>(std::ceil(std::log2(std::max(max_coeff, 1.0)))) + 1;
        if (max_coeff_bit_count >= total_bits || max_coeff_bit_count > 63)
            throw std::invalid_argument("encoded values are too large");
    }
    DeviceBuffer ews(he_encrypt_batch_workspace_words(h, L, (uint32_t)items));
    check_status(he_encrypt_batch(h, L, (uint32_t)items, pk.pk_.data(), context.prng_key(), context.next_stream(3 * items),
                                  batch.get(), ews.get(), st),
                 "he_encrypt_batch");
    // one ciphertext object per message, each a slice of the batch (no copies)
    std::vector<CAHELGPUCiphertext> out(items);
    auto shared = std::make_shared<DeviceBuffer>(std::move(batch));
    for (std::size_t k = 0; k < items; k++) {
        CAHELGPUCiphertext &ct = out[k];
        ct.adopt(DeviceBuffer::slice(shared, k * words, words));
        ct.size_ = 2;
        ct.coeff_modulus_size_ = L;
        ct.poly_modulus_degree_ = n;
        ct.chain_index_ = chain;
        ct.parms_id_ = context.parms_id_at(chain);
        ct.scale_ = scale;
        ct.is_ntt_form_ = true;
        ct.is_asymmetric_ = true;
    }
    return out;
}

void CAHELGPUCKKSEncoder::encode_complex(const CAHELGPUContext &context, const double *re, const double *im,
                                         std::size_t count, std::size_t chain_index, double scale,
                                         CAHELGPUPlaintext &destination) {
    const std::size_t n = context.poly_degree();
    if (count > slots_) throw std::invalid_argument("values_size is too large");
    const int total_bits = context.total_coeff_modulus_bit_count(chain_index);
    if (scale <= 0 || (static_cast<int>(std::log2(scale)) + 1 >= total_bits))
        throw std::invalid_argument("scale out of bounds");
    const std::size_t ss = message_slots(count);
    const uint32_t limbs = (uint32_t)context.limbs_at(chain_index);
    destination.resize(limbs, n);
    he_context *h = context.handle();
    DeviceBuffer ws(he_ckks_workspace_words(h, limbs));
    DeviceBuffer staging(2 * ss);  // the values, real parts then imaginary parts
    double *d_re = reinterpret_cast<double *>(staging.get());
    double *d_im = im ? d_re + ss : nullptr;
    if (count) {
        // (through page-locked memory, without waiting: the download of the largest coefficient below is the wait)
        double *host = pinned_stage((im ? 2 : 1) * count * sizeof(double));
        std::memcpy(host, re, count * sizeof(double));
        check_status(he_memcpy_h2d_async(d_re, host, count * sizeof(double), context.stream()), "upload");
        if (im) {
            std::memcpy(host + count, im, count * sizeof(double));
            check_status(he_memcpy_h2d_async(d_im, host + count, count * sizeof(double), context.stream()), "upload");
        }
    }
    check_status(he_ckks_encode(h, d_re, d_im, (uint32_t)count, (uint32_t)ss, scale, limbs, destination.data(),
                                ws.get(), context.stream()),
                 "he_ckks_encode");
    double max_coeff = 0.0;
    check_status(he_memcpy_d2h(&max_coeff, ws.get(), sizeof(double), context.stream()), "download");
    const int max_coeff_bit_count = static_cast<int>(std::ceil(std::log2(std::max(max_coeff, 1.0)))) + 1;
    if (max_coeff_bit_count >= total_bits) throw std::invalid_argument("encoded values are too large");
    if (max_coeff_bit_count > 63)
        throw std::invalid_argument("encoded values are too large: coefficients above 2^62 are not supported");
    destination.chain_index() = chain_index;
    destination.scale() = scale;
    destination.parms_id() = context.parms_id_at(chain_index);
    destination.is_ntt_form_ = true;
}

void CAHELGPUCKKSEncoder::encode(const CAHELGPUContext &context, const std::vector<double> &values,
                                 std::size_t chain_index, double scale, CAHELGPUPlaintext &destination) {
    encode_complex(context, values.data(), nullptr, values.size(), chain_index, scale, destination);
}

// the first `count` complex values of the decoding, interleaved (re, im), into v
void CAHELGPUCKKSEncoder::decode_values(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain,
                                        std::size_t count, std::vector<double> &v) {
    if (!plain.is_ntt_form()) throw std::invalid_argument("plain is not in NTT form");
    const uint32_t limbs = (uint32_t)plain.coeff_modulus_size();
    if (limbs == 0 || !plain.data()) throw std::invalid_argument("plain is empty");
    const int total_bits = context.total_coeff_modulus_bit_count(plain.chain_index());
    if (plain.scale() <= 0 || (static_cast<int>(std::log2(plain.scale())) >= total_bits))
        throw std::invalid_argument("scale out of bounds");
    if (sparse_slots_ == 0) sparse_slots_ = slots_;   // as the reference: decoding first fixes the full slot count
    const std::size_t ss = sparse_slots_;
    if (count == 0 || count > ss) count = ss;

    he_context *h = context.handle();
    DeviceBuffer ws(he_ckks_workspace_words(h, limbs));
    DeviceBuffer out(2 * ss);
    check_status(he_ckks_decode(h, plain.data(), limbs, (uint32_t)ss, plain.scale(),
                                reinterpret_cast<double *>(out.get()), ws.get(), context.stream()),
                 "he_ckks_decode");
    v.resize(2 * count);
    check_status(he_memcpy_d2h(v.data(), out.get(), v.size() * sizeof(double), context.stream()), "download");
}

void CAHELGPUCKKSEncoder::decode_complex(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain,
                                         std::vector<double> &re, std::vector<double> &im) {
    std::vector<double> v;
    decode_values(context, plain, 0, v);
    const std::size_t ss = v.size() / 2;
    re.resize(ss);
    im.resize(ss);
    for (std::size_t i = 0; i < ss; i++) {
        re[i] = v[2 * i];
        im[i] = v[2 * i + 1];
    }
}

void CAHELGPUCKKSEncoder::decode_prefix(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain,
                                        std::size_t count, std::vector<double> &destination) {
    std::vector<double> v;
    decode_values(context, plain, count, v);
    destination.resize(v.size() / 2);
    for (std::size_t i = 0; i < destination.size(); i++) destination[i] = v[2 * i];
}

void CAHELGPUCKKSEncoder::decode(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain,
                                 std::vector<double> &destination) {
    std::vector<double> im;
    decode_complex(context, plain, destination, im);
}
