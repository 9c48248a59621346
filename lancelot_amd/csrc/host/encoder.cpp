// CKKS encoder: slots <-> plaintext polynomial through the canonical embedding restricted to the orbit
// 5^j mod 2N (cahel-main/src/ckks.cu:34-209 encode, :292-465 decode; transform of src/fft.cu; rounding and
// residues of src/rns_base.cu:121-156; CRT composition of src/rns_base.cu:325-459).
//
// The special FFT (HEAAN's fftSpecial / fftSpecialInv butterfly network, FP64) and the CRT composition run
// on the host with OpenMP; residue decomposition and the NTTs run on the GPU.  Decoded values agree with
// the reference up to FP64 operation order (bounded by the 2^-20 acceptance tolerance), not bit for bit.
#include <cmath>
#include <complex>

#include "cahel.h"

using namespace cahel;
using cplx = std::complex<double>;

CAHELGPUCKKSEncoder::CAHELGPUCKKSEncoder(const CAHELGPUContext &context) {
    if (context.scheme() != scheme_type::ckks) throw std::invalid_argument("unsupported scheme");
    const std::size_t n = context.poly_degree(), m = 2 * n;
    slots_ = n >> 1;
    first_chain_index_ = context.get_first_index();
    rot_group_.resize(slots_);
    uint32_t pos = 1;
    for (std::size_t i = 0; i < slots_; i++) {
        rot_group_[i] = pos;
        pos = (uint32_t)(((uint64_t)pos * 5) & (m - 1));
    }
    ksi_re_.resize(m + 1);
    ksi_im_.resize(m + 1);
    const double pi = 3.14159265358979323846264338327950288;
    for (std::size_t k = 0; k <= m; k++) {
        const double angle = 2.0 * pi * (double)k / (double)m;
        ksi_re_[k] = std::cos(angle);
        ksi_im_[k] = std::sin(angle);
    }
}

namespace {

void bit_reverse_inplace(std::vector<cplx> &v) {
    const std::size_t size = v.size();
    int bits = 0;
    while (((std::size_t)1 << bits) < size) bits++;
    for (std::size_t i = 0; i < size; i++) {
        const std::size_t j = reverse_bits((uint32_t)i, bits);
        if (i < j) std::swap(v[i], v[j]);
    }
}

}  // namespace

void CAHELGPUCKKSEncoder::encode_complex(const CAHELGPUContext &context, const double *re, const double *im,
                                         std::size_t count, std::size_t chain_index, double scale,
                                         CAHELGPUPlaintext &destination) {
    const std::size_t n = context.poly_degree(), m = 2 * n;
    if (count > slots_) throw std::invalid_argument("values_size is too large");
    const int total_bits = context.total_coeff_modulus_bit_count(chain_index);
    if (scale <= 0 || (static_cast<int>(std::log2(scale)) + 1 >= total_bits))
        throw std::invalid_argument("scale out of bounds");
    if (sparse_slots_ == 0) {
        // the first message fixes the slot count for the lifetime of the encoder (src/ckks.cu:131-142)
        std::size_t s = 1;
        while (s < count) s <<= 1;
        sparse_slots_ = s;
    } else if (count > sparse_slots_) {
        throw std::invalid_argument("values_size exceeds previous message length");
    }
    if (sparse_slots_ < 2) throw std::invalid_argument("single value encoding is not available");
    const std::size_t ss = sparse_slots_;
    std::vector<cplx> v(ss, cplx(0.0, 0.0));
    for (std::size_t i = 0; i < count; i++) v[i] = cplx(re[i], im ? im[i] : 0.0);

    // inverse special FFT: decimation-in-frequency butterflies, then bit reversal, then scale / slots
    for (std::size_t len = ss; len >= 2; len >>= 1) {
        const std::size_t lenh = len >> 1, lenq = len << 2, gap = m / lenq;
#pragma omp parallel for if (ss >= 4096)
        for (std::size_t i = 0; i < ss; i += len) {
            for (std::size_t j = 0; j < lenh; j++) {
                const std::size_t idx = (lenq - (rot_group_[j] % lenq)) * gap;
                const cplx w(ksi_re_[idx], ksi_im_[idx]);
                const cplx u = v[i + j] + v[i + j + lenh];
                const cplx t = (v[i + j] - v[i + j + lenh]) * w;
                v[i + j] = u;
                v[i + j + lenh] = t;
            }
        }
    }
    bit_reverse_inplace(v);
    const double fix = scale / (double)ss;

    std::vector<double> coeffs(n, 0.0);
    const std::size_t gap = slots_ / ss;
    double max_coeff = 0.0;
    for (std::size_t i = 0; i < ss; i++) {
        const double a = std::round(v[i].real() * fix), b = std::round(v[i].imag() * fix);
        coeffs[i * gap] = a;
        coeffs[slots_ + i * gap] = b;
        max_coeff = std::max(max_coeff, std::max(std::fabs(a), std::fabs(b)));
    }
    const int max_coeff_bit_count = static_cast<int>(std::ceil(std::log2(std::max(max_coeff, 1.0)))) + 1;
    if (max_coeff_bit_count >= total_bits) throw std::invalid_argument("encoded values are too large");
    if (max_coeff_bit_count > 63)
        throw std::invalid_argument("encoded values are too large: coefficients above 2^62 are not supported");

    const uint32_t limbs = (uint32_t)context.limbs_at(chain_index);
    destination.resize(limbs, n);
    DeviceBuffer staging(n);  // N doubles
    he_context *h = context.handle();
    check_status(he_memcpy_h2d(staging.get(), coeffs.data(), n * sizeof(double), context.stream()), "upload");
    check_status(he_decompose_real(h, reinterpret_cast<const double *>(staging.get()), destination.data(), limbs, 0,
                                   context.stream()),
                 "he_decompose_real");
    check_status(he_ntt_forward(h, destination.data(), 1, limbs, limbs, 0, limbs, 0, context.stream()), "he_ntt_forward");
    destination.chain_index() = chain_index;
    destination.scale() = scale;
    destination.parms_id() = context.parms_id_at(chain_index);
    destination.is_ntt_form_ = true;
}

void CAHELGPUCKKSEncoder::encode(const CAHELGPUContext &context, const std::vector<double> &values,
                                 std::size_t chain_index, double scale, CAHELGPUPlaintext &destination) {
    encode_complex(context, values.data(), nullptr, values.size(), chain_index, scale, destination);
}

void CAHELGPUCKKSEncoder::decode_complex(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain,
                                         std::vector<double> &re, std::vector<double> &im) {
    if (!plain.is_ntt_form()) throw std::invalid_argument("plain is not in NTT form");
    const std::size_t n = context.poly_degree(), m = 2 * n;
    const uint32_t limbs = (uint32_t)plain.coeff_modulus_size();
    if (limbs == 0 || !plain.data()) throw std::invalid_argument("plain is empty");
    const int total_bits = context.total_coeff_modulus_bit_count(plain.chain_index());
    if (plain.scale() <= 0 || (static_cast<int>(std::log2(plain.scale())) >= total_bits))
        throw std::invalid_argument("scale out of bounds");
    if (sparse_slots_ == 0) sparse_slots_ = slots_;
    const std::size_t ss = sparse_slots_;

    he_context *h = context.handle();
    DeviceBuffer copy((std::size_t)limbs * n);
    check_status(he_memcpy_d2d(copy.get(), plain.data(), (std::size_t)limbs * n * sizeof(uint64_t), context.stream()), "copy");
    check_status(he_ntt_inverse(h, copy.get(), 1, limbs, limbs, 0, limbs, 0, context.stream()), "he_ntt_inverse");
    std::vector<uint64_t> res((std::size_t)limbs * n);
    check_status(he_memcpy_d2h(res.data(), copy.get(), res.size() * sizeof(uint64_t), context.stream()), "download");

    // CRT composition by Garner's mixed-radix form: v = d_0 + d_1 q_0 + d_2 q_0 q_1 + ...; centred around 0
    // using the mixed-radix digits of (Q - 1) / 2 (every q_i is odd, so those digits are (q_i - 1) / 2).
    const auto &mods = context.key_modulus();
    std::vector<uint64_t> q(limbs);
    for (uint32_t i = 0; i < limbs; i++) q[i] = mods[i].value();
    // inv[i][j] = q_j^-1 mod q_i for j < i
    std::vector<std::vector<uint64_t>> inv(limbs);
    for (uint32_t i = 0; i < limbs; i++)
        for (uint32_t j = 0; j < i; j++) inv[i].push_back(invert_mod(q[j] % q[i], q[i]));
    std::vector<double> qd(limbs);
    for (uint32_t i = 0; i < limbs; i++) qd[i] = (double)q[i];
    const double inv_scale = 1.0 / plain.scale();
    const std::size_t gap = slots_ / ss;
    std::vector<cplx> v(ss);
#pragma omp parallel
    {
        std::vector<uint64_t> d(limbs);
#pragma omp for
        for (std::size_t s = 0; s < 2 * ss; s++) {
            const std::size_t coeff = s < ss ? s * gap : slots_ + (s - ss) * gap;
            for (uint32_t i = 0; i < limbs; i++) {
                uint64_t t = res[(std::size_t)i * n + coeff];
                for (uint32_t j = 0; j < i; j++) {
                    const uint64_t dj = d[j] % q[i];
                    t = mul_mod(t >= dj ? t - dj : t + q[i] - dj, inv[i][j], q[i]);
                }
                d[i] = t;
            }
            // negative iff the digits, read from the top, exceed those of (Q-1)/2
            bool negative = false;
            for (uint32_t i = limbs; i-- > 0;) {
                const uint64_t h2 = (q[i] - 1) >> 1;
                if (d[i] != h2) {
                    negative = d[i] > h2;
                    break;
                }
            }
            if (negative) {
                // Q - v = (Q - 1 - v) + 1, digit-wise complement then increment
                for (uint32_t i = 0; i < limbs; i++) d[i] = q[i] - 1 - d[i];
                for (uint32_t i = 0; i < limbs; i++) {
                    if (++d[i] < q[i]) break;
                    d[i] = 0;
                }
            }
            double acc = 0.0;
            for (uint32_t i = limbs; i-- > 0;) acc = acc * qd[i] + (double)d[i];
            const double val = (negative ? -acc : acc) * inv_scale;
            if (s < ss)
                reinterpret_cast<double *>(&v[s])[0] = val;
            else
                reinterpret_cast<double *>(&v[s - ss])[1] = val;
        }
    }

    // forward special FFT: bit reversal, then decimation-in-time butterflies
    bit_reverse_inplace(v);
    for (std::size_t len = 2; len <= ss; len <<= 1) {
        const std::size_t lenh = len >> 1, lenq = len << 2, gapw = m / lenq;
#pragma omp parallel for if (ss >= 4096)
        for (std::size_t i = 0; i < ss; i += len) {
            for (std::size_t j = 0; j < lenh; j++) {
                const std::size_t idx = (rot_group_[j] % lenq) * gapw;
                const cplx w(ksi_re_[idx], ksi_im_[idx]);
                const cplx u = v[i + j];
                const cplx t = v[i + j + lenh] * w;
                v[i + j] = u + t;
                v[i + j + lenh] = u - t;
            }
        }
    }
    re.resize(ss);
    im.resize(ss);
    for (std::size_t i = 0; i < ss; i++) {
        re[i] = v[i].real();
        im[i] = v[i].imag();
    }
}

void CAHELGPUCKKSEncoder::decode(const CAHELGPUContext &context, const CAHELGPUPlaintext &plain,
                                 std::vector<double> &destination) {
    std::vector<double> im;
    decode_complex(context, plain, destination, im);
}
