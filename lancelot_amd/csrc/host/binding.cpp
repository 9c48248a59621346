// Python module pyCAHEL: the names, argument orders and defaults of cahel-main/python/src/binding.cu:8-156, so
// that lancelot-main-GPU/utils/byzantine_fl.py and ckks.py run against this engine unchanged.  Names that start
// with an underscore, and the accessor methods on context / plaintext / ciphertext / keys, are additions used
// by the test-suite and the benchmark (seeding, raw device pointers, host copies); they do not exist in the
// reference and nothing in Lancelot calls them.
#include <fstream>
#include <sstream>

#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include "cahel.h"

namespace py = pybind11;
using namespace cahel;

namespace {

py::array_t<uint64_t> to_host(const uint64_t *dev, std::vector<py::ssize_t> shape) {
    py::array_t<uint64_t> out(shape);
    std::size_t words = 1;
    for (auto s : shape) words *= (std::size_t)s;
    if (words) check_status(he_memcpy_d2h(out.mutable_data(), dev, words * sizeof(uint64_t), cahel::current_stream()), "download");
    return out;
}

// save / load / to_bytes / from_bytes on top of the C++ stream members (the reference binds none of them)
template <typename T, typename C>
void def_serialization(C &cls) {
    cls.def("save", [](const T &self, const std::string &path) {
           std::ofstream f(path, std::ios::binary | std::ios::trunc);
           if (!f) throw std::runtime_error("I/O error");
           self.save(f);
       })
        .def("load", [](T &self, const CAHELGPUContext &context, const std::string &path) {
            std::ifstream f(path, std::ios::binary);
            if (!f) throw std::runtime_error("I/O error");
            self.load(context, f);
        })
        .def("to_bytes", [](const T &self) {
            std::ostringstream s(std::ios::binary);
            self.save(s);
            return py::bytes(s.str());
        })
        .def("from_bytes", [](T &self, const CAHELGPUContext &context, const py::bytes &data) {
            std::istringstream s(std::string(data), std::ios::binary);
            self.load(context, s);
        });
}

py::tuple id_tuple(const parms_id_type &id) { return py::make_tuple(id[0], id[1], id[2], id[3]); }

}  // namespace

PYBIND11_MODULE(pyCAHEL, m) {
    m.doc() = "MI355X-native CKKS engine with the pyCAHEL interface";

    py::enum_<scheme_type>(m, "scheme_type")
        .value("none", scheme_type::none)
        .value("bgv", scheme_type::bgv)
        .value("bfv", scheme_type::bfv)
        .value("ckks", scheme_type::ckks)
        .export_values();
    py::enum_<mul_tech_type>(m, "mul_tech_type")
        .value("none", mul_tech_type::none)
        .value("behz", mul_tech_type::behz)
        .value("hps", mul_tech_type::hps)
        .value("hps_overq", mul_tech_type::hps_overq)
        .value("hps_overq_leveled", mul_tech_type::hps_overq_leveled)
        .export_values();
    py::enum_<sec_level_type>(m, "sec_level_type")
        .value("none", sec_level_type::none)
        .value("tc128", sec_level_type::tc128)
        .value("tc192", sec_level_type::tc192)
        .value("tc256", sec_level_type::tc256)
        .export_values();

    py::class_<Modulus>(m, "modulus").def(py::init<std::uint64_t>()).def("value", &Modulus::value);

    m.def("coeff_modulus_create", &CoeffModulus::Create);

    py::class_<EncryptionParameters>(m, "params")
        .def(py::init<scheme_type>())
        .def("set_mul_tech", &EncryptionParameters::set_mul_tech)
        .def("set_poly_modulus_degree", &EncryptionParameters::set_poly_modulus_degree)
        .def("set_special_modulus_size", &EncryptionParameters::set_special_modulus_size)
        .def("set_galois_elts", &EncryptionParameters::set_galois_elts)
        .def("set_coeff_modulus", &EncryptionParameters::set_coeff_modulus)
        .def("parms_id", [](const EncryptionParameters &p) { return id_tuple(p.parms_id()); })
        .def("poly_modulus_degree", &EncryptionParameters::poly_modulus_degree)
        .def("coeff_modulus", [](const EncryptionParameters &p) {
            std::vector<uint64_t> v;
            for (const auto &mod : p.coeff_modulus()) v.push_back(mod.value());
            return v;
        })
        .def("to_bytes", [](const EncryptionParameters &p) {
            std::ostringstream s(std::ios::binary);
            p.save(s);
            return py::bytes(s.str());
        })
        .def("from_bytes", [](EncryptionParameters &p, const py::bytes &data) {
            std::istringstream s(std::string(data), std::ios::binary);
            p.load(s);
        });
    m.def("_blake2b", [](const py::bytes &data, std::size_t digest_size) {
        const std::string in(data);
        std::string out(digest_size, '\0');
        blake2b(out.data(), digest_size, in.data(), in.size());
        return py::bytes(out);
    });

    py::class_<CAHELGPUContext>(m, "context")
        .def(py::init<EncryptionParameters &, bool, sec_level_type>())
        .def("set_seed", &CAHELGPUContext::set_seed)
        .def("he_handle", [](const CAHELGPUContext &c) { return reinterpret_cast<std::uintptr_t>(c.handle()); })
        .def("poly_degree", &CAHELGPUContext::poly_degree)
        .def("size_q", &CAHELGPUContext::size_q)
        .def("size_p", &CAHELGPUContext::size_p)
        .def("limbs_at", &CAHELGPUContext::limbs_at)
        .def("moduli", [](const CAHELGPUContext &c) {
            std::vector<uint64_t> v;
            for (auto &mo : c.key_modulus()) v.push_back(mo.value());
            return v;
        })
        .def("galois_elts", &CAHELGPUContext::galois_elts)
        .def("psi_table", [](const CAHELGPUContext &c) {
            return py::array_t<uint64_t>({(py::ssize_t)c.size_qp(), (py::ssize_t)c.poly_degree(), (py::ssize_t)2},
                                         c.psi_host().data());
        })
        .def("ipsi_table", [](const CAHELGPUContext &c) {
            return py::array_t<uint64_t>({(py::ssize_t)c.size_qp(), (py::ssize_t)c.poly_degree(), (py::ssize_t)2},
                                         c.ipsi_host().data());
        })
        .def("level_tables", [](const CAHELGPUContext &c, std::size_t L) {
            const auto &lh = c.level_host(L);
            py::dict d;
            d["beta"] = lh.beta;
            d["part_hat_inv"] = lh.part_hat_inv;
            d["digit_mats"] = lh.digit_mats;
            d["digit_mat_off"] = lh.digit_mat_off;
            d["qlast_inv"] = lh.qlast_inv;
            return d;
        });

    py::class_<CAHELGPUSecretKey>(m, "secret_key")
        .def(py::init<EncryptionParameters &>())
        .def("gen_secretkey", &CAHELGPUSecretKey::gen_secretkey)
        .def("gen_publickey", &CAHELGPUSecretKey::gen_publickey, py::arg("context"), py::arg("public_key"),
             py::arg("save_seed") = true)
        .def("gen_relinkey", &CAHELGPUSecretKey::gen_relinkey, py::arg("context"), py::arg("relin_key"),
             py::arg("save_seed") = false)
        .def("create_galois_keys", &CAHELGPUSecretKey::create_galois_keys, py::arg("context"), py::arg("galois_key"),
             py::arg("save_seed") = false)
        .def("encrypt_symmetric",
             py::overload_cast<const CAHELGPUContext &, const CAHELGPUPlaintext &, bool>(&CAHELGPUSecretKey::encrypt_symmetric,
                                                                                         py::const_))
        .def("decrypt", py::overload_cast<const CAHELGPUContext &, const CAHELGPUCiphertext &>(&CAHELGPUSecretKey::decrypt),
             py::call_guard<py::gil_scoped_release>())
        .def("set_noise_flooding", &CAHELGPUSecretKey::set_noise_flooding)
        .def("decrypt_decode_many",
             [](CAHELGPUSecretKey &k, const CAHELGPUContext &c, const std::vector<const CAHELGPUCiphertext *> &cts,
                std::size_t slots, std::size_t count) {
                 std::vector<double> out;
                 {
                     py::gil_scoped_release release;
                     out = k.decrypt_decode_many(c, cts, slots, count);
                 }
                 py::array_t<double> a({(py::ssize_t)cts.size(), (py::ssize_t)count});
                 std::copy(out.begin(), out.end(), a.mutable_data());
                 return a;
             },
             py::arg("context"), py::arg("ciphertexts"), py::arg("slots"), py::arg("count") = 1)
        .def("to_numpy", [](const CAHELGPUSecretKey &s, const CAHELGPUContext &c) {
            return to_host(s.secret_key_array(), {(py::ssize_t)c.size_qp(), (py::ssize_t)c.poly_degree()});
        });

    py::class_<CAHELGPUPublicKey>(m, "public_key")
        .def(py::init<CAHELGPUContext &>())
        .def("encrypt_asymmetric",
             py::overload_cast<const CAHELGPUContext &, const CAHELGPUPlaintext &, bool>(&CAHELGPUPublicKey::encrypt_asymmetric,
                                                                                         py::const_),
             py::arg("context"), py::arg("plaintext"), py::arg("save_seed") = false, py::call_guard<py::gil_scoped_release>())
        .def("to_numpy", [](const CAHELGPUPublicKey &k) {
            return to_host(k.pk_.data(), {(py::ssize_t)k.pk_.size(), (py::ssize_t)k.pk_.coeff_modulus_size(),
                                          (py::ssize_t)k.pk_.poly_modulus_degree()});
        });

    py::class_<CAHELGPURelinKey>(m, "relin_key")
        .def(py::init<CAHELGPUContext &>())
        .def("digit_count", [](const CAHELGPURelinKey &k) { return k.public_keys_.size(); })
        .def("copy", [](const CAHELGPURelinKey &k) { return CAHELGPURelinKey(k); })
        .def("digit_ptr", [](const CAHELGPURelinKey &k, std::size_t d) {
            return reinterpret_cast<std::uintptr_t>(k.public_keys_.at(d).pk_.data());
        })
        .def("digit_to_numpy", [](const CAHELGPURelinKey &k, std::size_t d) {
            const auto &c = k.public_keys_.at(d).pk_;
            return to_host(c.data(), {(py::ssize_t)c.size(), (py::ssize_t)c.coeff_modulus_size(),
                                      (py::ssize_t)c.poly_modulus_degree()});
        });

    py::class_<CAHELGPUGaloisKey>(m, "galois_key")
        .def(py::init<CAHELGPUContext &>())
        .def("key_count", [](const CAHELGPUGaloisKey &k) { return k.relin_keys_.size(); })
        .def("key", [](CAHELGPUGaloisKey &k, std::size_t i) -> CAHELGPURelinKey & { return k.relin_keys_.at(i); },
             py::return_value_policy::reference_internal);

    m.def("get_elts_from_steps", &get_elts_from_steps);

    py::class_<CAHELGPUCKKSEncoder>(m, "ckks_encoder")
        .def(py::init<CAHELGPUContext &>())
        .def("slot_count", &CAHELGPUCKKSEncoder::slot_count)
        .def("reset_sparse_slots", &CAHELGPUCKKSEncoder::reset_sparse_slots)
        // numpy fast paths (no per-element conversion); lists fall through to the reference's signatures
        .def("encode",
             [](CAHELGPUCKKSEncoder &e, const CAHELGPUContext &c, py::array_t<double, py::array::c_style> v, double scale) {
                 CAHELGPUPlaintext p(c);
                 const double *values = v.data();
                 const std::size_t count = (std::size_t)v.size();
                 py::gil_scoped_release release;
                 e.encode_complex(c, values, nullptr, count, e.first_chain_index(), scale, p);
                 return p;
             },
             py::arg("context"), py::arg("values").noconvert(), py::arg("scale"))
        .def("encode_to",
             [](CAHELGPUCKKSEncoder &e, const CAHELGPUContext &c, py::array_t<double, py::array::c_style> v,
                std::size_t chain_index, double scale) {
                 CAHELGPUPlaintext p(c);
                 e.encode_complex(c, v.data(), nullptr, (std::size_t)v.size(), chain_index, scale, p);
                 return p;
             },
             py::arg("context"), py::arg("values").noconvert(), py::arg("chain_index"), py::arg("scale"))
        .def("encode_encrypt_many",
             [](CAHELGPUCKKSEncoder &e, const CAHELGPUContext &c, const CAHELGPUPublicKey &pk,
                py::array_t<double, py::array::c_style> v, double scale) {
                 if (v.ndim() != 2) throw std::invalid_argument("values must be a two-dimensional array");
                 const double *values = v.data();
                 const std::size_t items = (std::size_t)v.shape(0), count = (std::size_t)v.shape(1);
                 py::gil_scoped_release release;
                 return e.encode_encrypt_many(c, pk, values, items, count, count, scale);
             },
             py::arg("context"), py::arg("public_key"), py::arg("values").noconvert(), py::arg("scale"))
        .def("decode_array",
             [](CAHELGPUCKKSEncoder &e, const CAHELGPUContext &c, const CAHELGPUPlaintext &p, std::size_t count) {
                 std::vector<double> out;
                 {
                     py::gil_scoped_release release;
                     e.decode_prefix(c, p, count, out);
                 }
                 return py::array_t<double>((py::ssize_t)out.size(), out.data());
             },
             py::arg("context"), py::arg("plain"), py::arg("count") = 0)
        .def("encode", py::overload_cast<const CAHELGPUContext &, const std::vector<double> &, double>(
                           &CAHELGPUCKKSEncoder::encode))
        .def("encode_to", py::overload_cast<const CAHELGPUContext &, const std::vector<double> &, std::size_t, double>(
                              &CAHELGPUCKKSEncoder::encode))
        .def("decode",
             py::overload_cast<const CAHELGPUContext &, const CAHELGPUPlaintext &>(&CAHELGPUCKKSEncoder::decode))
        .def("encode_complex",
             [](CAHELGPUCKKSEncoder &e, const CAHELGPUContext &c, const std::vector<std::complex<double>> &v,
                std::size_t chain_index, double scale) {
                 std::vector<double> re(v.size()), im(v.size());
                 for (std::size_t i = 0; i < v.size(); i++) {
                     re[i] = v[i].real();
                     im[i] = v[i].imag();
                 }
                 CAHELGPUPlaintext p(c);
                 e.encode_complex(c, re.data(), im.data(), v.size(), chain_index, scale, p);
                 return p;
             })
        .def("decode_complex", [](CAHELGPUCKKSEncoder &e, const CAHELGPUContext &c, const CAHELGPUPlaintext &p) {
            std::vector<double> re, im;
            e.decode_complex(c, p, re, im);
            std::vector<std::complex<double>> out(re.size());
            for (std::size_t i = 0; i < re.size(); i++) out[i] = {re[i], im[i]};
            return out;
        });

    py::class_<CAHELGPUPlaintext>(m, "plaintext")
        .def(py::init<>())
        .def(py::init<const CAHELGPUContext &>())
        .def("chain_index", [](const CAHELGPUPlaintext &p) { return p.chain_index(); })
        .def("scale", [](const CAHELGPUPlaintext &p) { return p.scale(); })
        .def("data_ptr", [](const CAHELGPUPlaintext &p) { return reinterpret_cast<std::uintptr_t>(p.data()); })
        .def("to_numpy", [](const CAHELGPUPlaintext &p) {
            return to_host(p.data(), {(py::ssize_t)p.coeff_modulus_size(), (py::ssize_t)p.poly_modulus_degree()});
        });

    py::class_<CAHELGPUCiphertext>(m, "ciphertext")
        .def(py::init<>())
        .def(py::init<const CAHELGPUContext &>())
        .def("set_scale", &CAHELGPUCiphertext::set_scale)
        .def("scale", [](const CAHELGPUCiphertext &c) { return c.scale(); })
        .def("size", &CAHELGPUCiphertext::size)
        .def("chain_index", [](const CAHELGPUCiphertext &c) { return c.chain_index(); })
        .def("coeff_modulus_size", &CAHELGPUCiphertext::coeff_modulus_size)
        .def("data_ptr", [](const CAHELGPUCiphertext &c) { return reinterpret_cast<std::uintptr_t>(c.data()); })
        .def("copy", [](const CAHELGPUCiphertext &c) { return CAHELGPUCiphertext(c); })
        // True between a relinearize_inplace whose key switch was deferred and the first use of the data
        .def("_has_pending_key_switch", &CAHELGPUCiphertext::has_pending_key_switch)
        .def("to_numpy", [](const CAHELGPUCiphertext &c) {
            return to_host(c.data(), {(py::ssize_t)c.size(), (py::ssize_t)c.coeff_modulus_size(),
                                      (py::ssize_t)c.poly_modulus_degree()});
        });

    // The evaluator only enqueues device work and touches no Python state: the interpreter lock is released so
    // that several Python threads, each on its own lane, can issue independent pipelines concurrently.
    const py::call_guard<py::gil_scoped_release> nogil;
    m.def("negate", &negate, nogil);
    m.def("negate_inplace", &negate_inplace, nogil);
    m.def("add", &add, nogil);
    m.def("add_inplace", &add_inplace, nogil);
    m.def("add_plain", &add_plain, nogil);
    m.def("add_plain_inplace", &add_plain_inplace, nogil);
    m.def("add_many", &add_many, nogil);
    m.def("sub", &sub, nogil);
    m.def("sub_inplace", &sub_inplace, py::arg("context"), py::arg("encrypted1"), py::arg("encrypted2"),
          py::arg("negate") = false, nogil);
    m.def("sub_plain", &sub_plain, nogil);
    m.def("sub_plain_inplace", &sub_plain_inplace, nogil);
    m.def("multiply", &multiply, nogil);
    m.def("multiply_inplace", &multiply_inplace, nogil);
    m.def("multiply_and_relin_inplace", &multiply_and_relin_inplace, nogil);
    m.def("multiply_plain", &multiply_plain, nogil);
    m.def("multiply_plain_inplace", &multiply_plain_inplace, nogil);
    m.def("multiply_many", &multiply_many, nogil);
    m.def("square", &square, nogil);
    m.def("square_inplace", &square_inplace, nogil);
    m.def("exponentiate", &exponentiate, nogil);
    m.def("exponentiate_inplace", &exponentiate_inplace, nogil);
    m.def("relinearize", &relinearize, nogil);
    m.def("relinearize_inplace", &relinearize_inplace, nogil);
    m.def("relinearize_rescale_inplace", &relinearize_rescale_inplace, nogil);
    m.def("multiply_relin_rescale", &multiply_relin_rescale, nogil);
    m.def("pair_square_distances", &pair_square_distances, py::arg("context"), py::arg("clients"), py::arg("pairs"),
          py::arg("relin_key"), py::arg("galois_key"), py::arg("rounds"), py::arg("scale") = 0.0, py::arg("drop_levels") = 0,
          nogil);
    m.def("mod_switch_to", py::overload_cast<const CAHELGPUContext &, const CAHELGPUPlaintext &, CAHELGPUPlaintext &, std::size_t>(&mod_switch_to), nogil);
    m.def("mod_switch_to", py::overload_cast<const CAHELGPUContext &, const CAHELGPUCiphertext &, CAHELGPUCiphertext &, std::size_t>(&mod_switch_to), nogil);
    m.def("mod_switch_to_inplace", py::overload_cast<const CAHELGPUContext &, CAHELGPUPlaintext &, std::size_t>(&mod_switch_to_inplace), nogil);
    m.def("mod_switch_to_inplace", py::overload_cast<const CAHELGPUContext &, CAHELGPUCiphertext &, std::size_t>(&mod_switch_to_inplace), nogil);
    m.def("mod_switch_to_next", py::overload_cast<const CAHELGPUContext &, const CAHELGPUPlaintext &, CAHELGPUPlaintext &>(&mod_switch_to_next), nogil);
    m.def("mod_switch_to_next", py::overload_cast<const CAHELGPUContext &, const CAHELGPUCiphertext &, CAHELGPUCiphertext &>(&mod_switch_to_next), nogil);
    m.def("mod_switch_to_next_inplace", py::overload_cast<const CAHELGPUContext &, CAHELGPUPlaintext &>(&mod_switch_to_next_inplace), nogil);
    m.def("mod_switch_to_next_inplace", py::overload_cast<const CAHELGPUContext &, CAHELGPUCiphertext &>(&mod_switch_to_next_inplace), nogil);
    m.def("rescale_to_next", &rescale_to_next, nogil);
    m.def("rescale_to_next_inplace", &rescale_to_next_inplace, nogil);
    m.def("apply_galois", &apply_galois, nogil);
    m.def("apply_galois_inplace", &apply_galois_inplace, nogil);
    m.def("rotate_rows", &rotate_rows, nogil);
    m.def("rotate_rows_inplace", &rotate_rows_inplace, nogil);
    m.def("rotate_columns", &rotate_columns, nogil);
    m.def("rotate_columns_inplace", &rotate_columns_inplace, nogil);
    m.def("rotate_vector", &rotate_vector, nogil);
    m.def("rotate_vector_inplace", &rotate_vector_inplace, nogil);
    m.def("hoisting", &hoisting, nogil);
    m.def("hoisting_inplace", &hoisting_inplace, nogil);
    m.def("complex_conjugate", &complex_conjugate, nogil);
    m.def("complex_conjugate_inplace", &complex_conjugate_inplace, nogil);

    m.def("_naf", &naf);
    m.def("_get_primes", &get_primes);
    m.def("_minimal_primitive_root", [](uint64_t degree, uint64_t q) {
        uint64_t r;
        if (!try_minimal_primitive_root(degree, q, r)) throw std::invalid_argument("no primitive root");
        return r;
    });
    m.def("_trim_pool", &DeviceBuffer::trim_pool);
    m.def("_synchronize", []() { cahel::synchronize_lanes(); });
    m.def("_set_lane", &cahel::set_lane);
    m.def("_current_lane", &cahel::current_lane);
    m.def("_lane_count", &cahel::lane_count);

    // serialization in the reference's byte layout, and the identifiers it carries
    {
        auto plain = py::reinterpret_borrow<py::class_<CAHELGPUPlaintext>>(m.attr("plaintext"));
        auto cipher = py::reinterpret_borrow<py::class_<CAHELGPUCiphertext>>(m.attr("ciphertext"));
        auto pk = py::reinterpret_borrow<py::class_<CAHELGPUPublicKey>>(m.attr("public_key"));
        auto rlk = py::reinterpret_borrow<py::class_<CAHELGPURelinKey>>(m.attr("relin_key"));
        auto glk = py::reinterpret_borrow<py::class_<CAHELGPUGaloisKey>>(m.attr("galois_key"));
        def_serialization<CAHELGPUPlaintext>(plain);
        def_serialization<CAHELGPUCiphertext>(cipher);
        def_serialization<CAHELGPUPublicKey>(pk);
        def_serialization<CAHELGPURelinKey>(rlk);
        def_serialization<CAHELGPUGaloisKey>(glk);
        plain.def("parms_id", [](const CAHELGPUPlaintext &p) { return id_tuple(p.parms_id()); });
        cipher.def("parms_id", [](const CAHELGPUCiphertext &c) { return id_tuple(c.parms_id()); });
        auto context = py::reinterpret_borrow<py::class_<CAHELGPUContext>>(m.attr("context"));
        context.def("parms_id_at", [](const CAHELGPUContext &c, std::size_t i) { return id_tuple(c.parms_id_at(i)); });
    }
}
