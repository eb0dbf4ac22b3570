// A driver written the way the reference's test programs are (test/HyraxTest.cu, test/tlookupTest.cu,
// the matmul block of test/llm.cu), against the host classes of this build: generators and table,
// integer and field-element commitments, opening with a real verification, a matmul sumcheck and a
// range lookup.  Compiled with g++ and linked with libgrape_host / libgrape_hip by the tests; prints
// "driver_flow OK" when every check holds.
#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <string>
#include <vector>
#include "../../include/grape_hip.h"
#include "../../grape_amd/host/ec_operation.hpp"
#include "../../grape_amd/host/fr_tensor.hpp"
#include "../../grape_amd/host/hyrax.hpp"
#include "../../grape_amd/host/ioutils.hpp"
#include "../../grape_amd/host/polynomial.hpp"
#include "../../grape_amd/host/prove.hpp"
#include "../../grape_amd/host/timer.hpp"
#include "../../grape_amd/host/tlookup.hpp"

static void require(bool ok, const char* what) {
    if (!ok) throw std::runtime_error(std::string("driver_flow: ") + what);
}

int main(int argc, char** argv) {
    const std::string dir = argc > 1 ? argv[1] : "/tmp";
    try {
        Fr::seed(2024);
        Timer timer;
        timer.start();
        const uint npoints = 1024, layer_num = 1, N = 4, com_scale = 16;   // rows of N * com_scale = 64
        affine_t* points = nullptr;
        require(grape_malloc((void**)&points, sizeof(affine_t) * 256 * npoints) == 0, "grape_malloc");
        std::vector<bn128> cpu_points = precompute_generators(npoints, 256, points);
        require(cpu_points.size() == npoints, "generator count");
        savebin(dir + "/points.bin", points, sizeof(affine_t) * 256 * npoints);          // test/ppgen.cu writes this file
        require(findsize(dir + "/points.bin") == sizeof(affine_t) * 256 * npoints, "points.bin size");

        // ---- commitments of an int tensor and of the same values as field elements agree (test/HyraxTest.cu:57-67)
        const uint size = 64 * 8;
        int* tensor = nullptr;
        generate_data(&tensor, size);
        Hyrax hyrax(layer_num, npoints / com_scale, points, cpu_points[0]);
        FrTensor fr_tensor(size, tensor);
        jacob_t* com_int = hyrax.commit(tensor, size, N);
        jacob_t* com_fr = hyrax.commit(fr_tensor, size, N);
        const uint rows = size / N / com_scale;
        std::vector<bn128> h_int(rows), h_fr(rows);
        require(grape_memcpy_d2h(h_int.data(), com_int, sizeof(jacob_t) * rows, nullptr) == 0, "d2h");
        require(grape_memcpy_d2h(h_fr.data(), com_fr, sizeof(jacob_t) * rows, nullptr) == 0, "d2h");
        for (uint i = 0; i < rows; i++) require(h_int[i] == h_fr[i], "int path and Fr path commit to different points");

        // ---- the same under a table budget that leaves only the small tables: int16 values go through
        // the two-digit table, field elements through the reference-format table; same commitments
        {
            std::vector<int> small(size);
            for (uint i = 0; i < size; i++) small[i] = (int)((i * 2654435761u) >> 16) % 65536 - 32768;
            small[0] = -32768; small[1] = 32767; small[2] = 0;
            int* d_small = nullptr;
            require(grape_malloc((void**)&d_small, sizeof(int) * size) == 0, "grape_malloc");
            require(grape_memcpy_h2d(d_small, small.data(), sizeof(int) * size, nullptr) == 0, "h2d");
            Hyrax tight(layer_num, npoints / com_scale, points, cpu_points[0]);
            tight.set_table_budget((size_t)8 << 20);        // 8 MiB: 2 * 256 * 64 entries of 128 bytes fit, 32768 * 64 do not
            FrTensor fr_small(size, d_small);
            jacob_t* c1 = tight.commit(d_small, size, N);
            jacob_t* c2 = tight.commit(fr_small, size, N);
            jacob_t* c3 = hyrax.commit(d_small, size, N);
            std::vector<bn128> h1(rows), h2(rows), h3(rows);
            require(grape_memcpy_d2h(h1.data(), c1, sizeof(jacob_t) * rows, nullptr) == 0, "d2h");
            require(grape_memcpy_d2h(h2.data(), c2, sizeof(jacob_t) * rows, nullptr) == 0, "d2h");
            require(grape_memcpy_d2h(h3.data(), c3, sizeof(jacob_t) * rows, nullptr) == 0, "d2h");
            for (uint i = 0; i < rows; i++) require(h1[i] == h2[i] && h1[i] == h3[i], "commitments differ between table choices");
            grape_free(c1); grape_free(c2); grape_free(c3); grape_free(d_small);
        }

        // ---- open at a random point, verify, and compare with the multilinear extension (test/HyraxTest.cu:76-125)
        std::vector<Fr> eval_point = random_vec(Log2(size));
        Fr c = Fr::random_element();
        FrTensor copy1(fr_tensor), copy2(fr_tensor);
        Hyrax_proof proof = hyrax.open(copy1, eval_point, c, size, N);
        require(hyrax.verify(proof, com_fr, eval_point, c, size, N), "opening does not verify");
        hyrax.verify(proof, com_fr, c, size, N);          // the reference's signature (include/Hyrax.cuh:85): throws on a mismatch
        {
            Hyrax_proof forged(proof);
            forged.result += Fr::one();
            bool refused = false;
            try {
                hyrax.verify(forged, com_fr, c, size, N);
            } catch (const std::runtime_error&) {
                refused = true;
            }
            require(refused, "a forged opening passed the reference-signature verify");
        }
        require(proof.result == copy2(eval_point), "opened value differs from the multilinear extension");

        // ---- matmul sumcheck (the pattern of test/llm.cu): Y[n][m] = sum_k A[n][k] B[m][k]
        const int Ln = 1, Nn = 8, Mn = 4, Kn = 16;
        FrTensor A = FrTensor::random(Ln * Nn * Kn), B = FrTensor::random(Ln * Mn * Kn);
        std::vector<Fr> hA = A.to_host(), hB = B.to_host(), hY((size_t)Nn * Mn);
        for (int n = 0; n < Nn; n++)
            for (int m = 0; m < Mn; m++) {
                Fr s = Fr::zero();
                for (int k = 0; k < Kn; k++) s += hA[n * Kn + k] * hB[m * Kn + k];
                hY[n * Mn + m] = s;
            }
        FrTensor Y = FrTensor::from_host(hY);
        std::vector<Fr> u = random_vec(Log2(Ln * Nn * Mn)), v = random_vec(Log2(Kn) + Log2(Ln));
        Fr claim = Y(u);
        SumcheckTranscript tr;
        std::pair<Fr, Fr> ab = prove_matmul(A, B, Ln, Nn, Mn, Kn, u, v, claim, &tr);
        require(tr.rounds.size() == Log2(Kn), "round count");
        require(ab.first * ab.second == claim, "A(v) * B(v) != final claim");

        // ---- range lookup (test/tlookupTest.cu): every value lies in [-512, 512)
        const uint D = 4096;
        std::vector<int> h_s(D);
        for (uint i = 0; i < D; i++) h_s[i] = (int)((i * 37 + 11) % 1024) - 512;
        int* d_s = nullptr;
        require(grape_malloc((void**)&d_s, sizeof(int) * D) == 0, "grape_malloc");
        require(grape_memcpy_h2d(d_s, h_s.data(), sizeof(int) * D, nullptr) == 0, "h2d");
        FrTensor S(D, d_s), S_keep(D, d_s), Aux(D);
        tLookupRange rs(-512, 1024);
        std::vector<Fr> v2 = random_vec(Log2(D));
        double commit_time = 0.0;
        Fr lookup_value = rs.prove(S, Aux, v2, hyrax, N, commit_time);
        require(lookup_value == S_keep(v2), "lookup value differs from S(v)");
        // ---- the reference's round-by-round entry points (src/tlookup.cu:117-244) on the same witness,
        // point and challenges: the same round polynomials and the same returned value as prove()
        {
            const uint Nt = rs.T.size;
            std::vector<Fr> u = random_vec(Log2(D));
            rs.set_u(u);
            FrTensor S1(D, d_s), A1(D);
            const Fr fused_value = rs.prove(S1, A1, v2, hyrax, N, commit_time);
            const SumcheckTranscript fused = rs.last_transcript;
            require(fused.rounds.size() == Log2(D), "lookup round count");
            FrTensor S2(D, d_s), A2(D);
            A2 = S2;
            A2 += (int)Nt;                      // beta is the table size (src/tlookup.cu:247)
            A2.inverse();
            FrTensor Bm(rs.B);
            Bm *= rs.m;
            const Fr alpha_sq = rs.alpha * rs.alpha;
            const Fr C = alpha_sq - Bm.sum(Nt);
            const Fr first_claim = rs.alpha + alpha_sq;
            const Fr N_div_D = Fr((long)Nt) * Fr((long)D).invert();
            const std::vector<Fr> v_hi(v2.begin() + Log2(Nt), v2.end()), v_lo(v2.begin(), v2.begin() + Log2(Nt));
            const Polynomial first = tLookup_phase1_step_poly(first_claim, A2, S2, rs.alpha, rs.beta, C, u);
            require(first.coefficients() == fused.rounds[0].coefficients(), "first round polynomial of the unfused form differs");
            const Fr unfused_value = tLookup_phase1(first_claim, A2, S2, rs.B, rs.T, rs.m, rs.alpha, rs.beta, C, N_div_D, alpha_sq, u, v_hi, v_lo);
            require(unfused_value == fused_value, "round-by-round lookup value differs from prove()");
        }

        // a witness with one value outside the range is rejected by the prover's own check
        h_s[5] = 600;
        require(grape_memcpy_h2d(d_s, h_s.data(), sizeof(int) * D, nullptr) == 0, "h2d");
        FrTensor S_bad(D, d_s);
        bool rejected = false;
        try {
            rs.prove(S_bad, Aux, v2, hyrax, N, commit_time);
        } catch (const std::runtime_error&) {
            rejected = true;
        }
        require(rejected, "out-of-range witness was not rejected");

        // ---- a lookup object outlives the Hyrax object whose table it holds: with another Hyrax object
        // (other generators, possibly at the same address) it builds its table again, and the commitment
        // of A it leaves is the new object's commitment of 1/(S + beta)
        {
            h_s[5] = (int)((5 * 37 + 11) % 1024) - 512;
            require(grape_memcpy_h2d(d_s, h_s.data(), sizeof(int) * D, nullptr) == 0, "h2d");
            tLookupRange kept(-512, 1024);
            {
                Hyrax first(layer_num, npoints / com_scale, points, cpu_points[0]);
                FrTensor Sa(D, d_s), Aa(D);
                kept.prove(Sa, Aa, v2, first, N, commit_time);
            }
            affine_t* points2 = nullptr;
            require(grape_malloc((void**)&points2, sizeof(affine_t) * 256 * npoints) == 0, "grape_malloc");
            std::vector<bn128> cpu_points2 = precompute_generators(npoints, 256, points2);
            require(!(cpu_points2[0] == cpu_points[0]), "second generator set equals the first");
            {
                Hyrax second(layer_num, npoints / com_scale, points2, cpu_points2[0]);
                FrTensor Sb(D, d_s), Ab(D);
                kept.prove(Sb, Ab, v2, second, N, commit_time);
                FrTensor A_ref(D, d_s);
                A_ref += 1024;                  // beta is the table size
                A_ref.inverse();
                affine_t* want = second.commit_affine(A_ref, D, N);
                const uint arows = D / N / com_scale;
                require(kept.com_A_rows == arows, "rows of com(A)");
                std::vector<unsigned char> got_b(sizeof(affine_t) * arows), want_b(sizeof(affine_t) * arows);
                require(grape_memcpy_d2h(got_b.data(), kept.com_A, got_b.size(), nullptr) == 0, "d2h");
                require(grape_memcpy_d2h(want_b.data(), want, want_b.size(), nullptr) == 0, "d2h");
                require(got_b == want_b, "com(A) after the Hyrax object changed is not the new object's commitment");
                grape_free(want);
            }
            grape_free(points2);
        }

        // ---- Fr_partial_me: the fold without compaction leaves value (o, g) at o * c * w + g
        {
            const uint c = 6, w = 5, outer = 3, n = outer * c * w;     // an odd tail in the second round
            FrTensor t = FrTensor::random(n), t2(t);
            std::vector<Fr> x = random_vec(Log2(c));
            fr_t* dx = grape_host::upload(x);
            t2.partial_eval(n, dx, c, 0, w);
            Fr_partial_me(n, t, dx, 0, c, w);
            const std::vector<Fr> strided = t.to_host(), compact = t2.to_host();
            for (uint o = 0; o < outer; o++)
                for (uint g = 0; g < w; g++) require(strided[o * c * w + g] == compact[o * w + g], "Fr_partial_me position");
            grape_free(dx);
        }

        grape_free(d_s);
        grape_free(com_int);
        grape_free(com_fr);
        grape_free(tensor);
        grape_free(points);
        timer.stop("driver_flow");
        std::printf("driver_flow OK\n");
        return 0;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "%s\n", e.what());
        return 1;
    }
}
