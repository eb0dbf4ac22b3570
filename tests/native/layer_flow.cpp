// One transformer block proved in the order of the reference's layer driver (test/llm.cu:73-611),
// written against the host classes of this build and fed by its own witness generator instead of
// the reference's data files: every remainder goes through a range lookup and an opening that must
// agree, every matrix product and element product through its sumcheck, the two tables through
// mapping lookups, claims on shared tensors are merged with combine_claims, and the claims are
// chained backwards from the block's output to its input exactly as the reference chains them.
// Any inconsistency throws.  Arguments: input_tokens (default 1024, a multiple of 16 and at least
// 1024 so that the softmax tensors cover the 2^20-entry exponential table).
//
// Compiled with g++ and linked with libgrape_host / libgrape_hip by the tests; prints
// "layer_flow OK" when every check holds.
#include <chrono>
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
#include "../../grape_amd/host/prove.hpp"
#include "../../grape_amd/host/tlookup.hpp"
#include "../../grape_amd/host/witness.hpp"

static void require(bool ok, const std::string& what) {
    if (!ok) throw std::runtime_error("layer_flow: " + what);
}

// seeded, roughly normal integers (sum of four uniforms) of standard deviation sigma
struct Rng {
    unsigned long long s;
    explicit Rng(unsigned long long seed) : s(seed * 0x9e3779b97f4a7c15ull + 1) {}
    unsigned next() {
        s ^= s << 13; s ^= s >> 7; s ^= s << 17;
        return (unsigned)(s >> 32);
    }
    int gauss(double sigma) {
        double u = 0;
        for (int i = 0; i < 4; i++) u += (double)next() / 4294967296.0;
        return (int)((u - 2.0) * 1.7320508 * sigma);      // variance of the sum of four uniforms is 1/3
    }
};

static int* device_ints(size_t n, Rng& rng, double sigma, int clip) {
    std::vector<int> h(n);
    for (size_t i = 0; i < n; i++) {
        int v = rng.gauss(sigma);
        if (clip) v = v < -clip ? -clip : (v > clip - 1 ? clip - 1 : v);
        h[i] = v;
    }
    int* d = nullptr;
    require(grape_malloc((void**)&d, sizeof(int) * n) == 0, "grape_malloc");
    require(grape_memcpy_h2d(d, h.data(), sizeof(int) * n, nullptr) == 0, "h2d");
    return d;
}

static int* upload(const std::vector<int>& h) {
    int* d = nullptr;
    require(grape_malloc((void**)&d, sizeof(int) * h.size()) == 0, "grape_malloc");
    require(grape_memcpy_h2d(d, h.data(), sizeof(int) * h.size(), nullptr) == 0, "h2d");
    return d;
}

static void write_table(const std::string& path, const std::vector<int>& t) {
    FILE* f = std::fopen(path.c_str(), "wb");
    require(f != nullptr, "cannot write " + path);
    require(std::fwrite(t.data(), sizeof(int), t.size(), f) == t.size(), "short write");
    std::fclose(f);
}

int main(int argc, char** argv) {
    const uint input_tokens = argc > 1 ? (uint)std::atoi(argv[1]) : 1024;
    const std::string tmp_dir = argc > 2 ? argv[2] : "/tmp";
    const uint dim = 4096, max_embed_dim = 11008, npoints = 16384, com_scale = 16, layer_num = 1;   // test/llm.cu:17-20
    try {
        require(input_tokens >= 1024 && input_tokens % 16 == 0, "input_tokens must be a multiple of 16, at least 1024");
        auto t_start = std::chrono::steady_clock::now();
        Fr::seed(777);
        // ---- public parameters (test/ppgen.cu): generators and the reference-format table
        affine_t* points = nullptr;
        require(grape_malloc((void**)&points, sizeof(affine_t) * 256 * (size_t)npoints * com_scale) == 0, "grape_malloc");
        std::vector<bn128> cpu_points = precompute_generators(npoints * com_scale, 256, points);
        Hyrax hyrax(layer_num, npoints, points, cpu_points[0]);

        // ---- weights, input, tables; the witness (zzllama/llama/model.py's tensors)
        Rng rng(2024);
        const size_t DD = (size_t)dim * dim, FD = (size_t)max_embed_dim * dim, TD = (size_t)input_tokens * dim;
        LayerWitness::Weights w;
        w.Q = device_ints(DD, rng, 1024, 32768);
        w.K = device_ints(DD, rng, 1024, 32768);
        w.V = device_ints(DD, rng, 1024, 32768);
        w.O = device_ints(DD, rng, 1024, 32768);
        w.gate = device_ints(FD, rng, 1024, 32768);
        w.up = device_ints(FD, rng, 1024, 32768);
        w.down = device_ints(FD, rng, 1024, 32768);
        w.norm_first = upload(std::vector<int>(dim, 65536));
        w.norm_second = upload(std::vector<int>(dim, 65536));
        int* x = device_ints(TD, rng, 65536, 0);
        const std::vector<int> exp_table = LayerWitness::make_exp_table(), silu_table = LayerWitness::make_silu_table();
        write_table(tmp_dir + "/exp-table.bin", exp_table);
        write_table(tmp_dir + "/swiglu-table.bin", silu_table);
        LayerWitness::Tables tables{upload(exp_table), upload(silu_table)};
        LayerWitness lw(input_tokens, dim, max_embed_dim);
        lw.generate(x, w, tables);
        std::printf("witness ready after %.1f s\n", std::chrono::duration<double>(std::chrono::steady_clock::now() - t_start).count());
        std::fflush(stdout);

        // ---- lookup objects (test/llm.cu:55-64)
        const uint SCALE1 = 1u << 16, SCALE2 = 1u << 20;
        tLookupRange rs(-(int)(SCALE1 / 2), SCALE1);
        tLookupRange swiglu_rs(-(1 << 19), 1 << 20);
        tLookupRange softmax_range_relation(0, 1 << 16);
        tLookupRangeMapping swiglu(-(1 << 18), 1 << 19, tmp_dir + "/swiglu-table.bin");
        tLookupRangeMapping exp(-(1 << 20) + 1, 1 << 20, tmp_dir + "/exp-table.bin");

        FrTensor tensor1(layer_num * dim * max_embed_dim), tensor2(layer_num * dim * max_embed_dim);
        FrTensor tensor3(layer_num * input_tokens * (1u << Log2(max_embed_dim))), tmp_tensor(layer_num * input_tokens * dim);
        std::vector<Fr> eval_point1, eval_point2, eval_point3, skip_eval_point;
        const Fr c = Fr::random_element();
        double commit_time = 0;
        int steps = 0;
        auto T = [&](const char* name) { return const_cast<int*>(lw.tensor(name)); };
        auto S = [&](const char* name) { return (uint)lw.tensor_size(name); };
        auto done = [&](const char* what) {
            steps++;
            std::printf("  %-28s ok (%.1f s)\n", what, std::chrono::duration<double>(std::chrono::steady_clock::now() - t_start).count());
            std::fflush(stdout);
        };
        // a remainder tensor: range proof at `point`, opening of the same tensor at `point`, both must agree
        auto remainder = [&](const char* name, tLookupRange& range, const std::vector<Fr>& point, uint msm_size, uint open_N) {
            const uint size = S(name);
            tensor1.get_data(size, T(name));
            tensor3.set_size(size);
            tensor3 = tensor1;
            const Fr value = range.prove(tensor1, tensor2, point, hyrax, msm_size, commit_time);
            Hyrax_proof pr = hyrax.open(tensor3, point, c, size, open_N);
            require(pr.result == value, std::string("lookup and opening disagree on ") + name);
            return value;
        };
        // a weight matrix product: sumcheck, then the weight's opening at the reassembled point
        auto weight_matmul = [&](const char* act, const char* weight, FrTensor* keep_act, uint N, uint M, uint K, std::vector<Fr>& u,
                                 std::vector<Fr>& v, Fr claim) {
            const uint sa = S(act), sw = S(weight);
            generate_random_eval_points((size_t)K * layer_num, v);
            tensor3.get_data(sa, T(act));
            tensor2.get_data(sw, T(weight));
            tensor1.set_size(sw);
            tensor1 = tensor2;
            if (keep_act) *keep_act = tensor3;
            std::pair<Fr, Fr> pr = prove_matmul(tensor3, tensor2, layer_num, N, M, K, u, v, claim);
            ReassembleVectors(u, v, Log2(N), Log2(K), Log2(M));
            Hyrax_proof op = hyrax.open(tensor1, v, c, sw, K);
            require(op.result == pr.second, std::string("weight opening disagrees with the sumcheck of W/") + weight);
            return pr;
        };

        // ======================= feed-forward, walking backwards (test/llm.cu:73-262) =======================
        uint size1 = S("Q/output");
        tensor1.get_data(size1, T("Q/output"));
        generate_random_eval_points(size1, eval_point1);
        Hyrax_proof proof = hyrax.open(tensor1, eval_point1, c, size1, size1 / layer_num / input_tokens);
        tensor1.get_data(S("Q/down_out"), T("Q/down_out"));
        Fr down_out_value = tensor1(eval_point1);
        skip_eval_point = eval_point1;
        Fr skip_value = proof.result - down_out_value;
        done("output = skip + down_out");

        Fr lookup_value = remainder("R/down_out", rs, eval_point1, dim, dim);
        down_out_value = down_out_value * Fr((long)SCALE1) + lookup_value;
        done("down_out remainder");

        std::pair<Fr, Fr> down_pair = weight_matmul("Q/upSilu", "W/down", nullptr, input_tokens, dim, max_embed_dim, eval_point1, eval_point2, down_out_value);
        Fr upSilu_value = down_pair.first;
        done("down projection");

        lookup_value = remainder("R/upSilu", rs, eval_point1, npoints, max_embed_dim);
        upSilu_value = upSilu_value * Fr((long)SCALE1) + lookup_value;
        done("upSilu remainder");

        size1 = S("Q/up_out");
        uint size2 = S("Q/silu_out");
        tensor1.get_data(size1, T("Q/up_out"));
        tensor2.get_data(size2, T("Q/silu_out"));
        generate_random_eval_points(size2, eval_point2);
        tensor3.set_size(size2);
        tensor3 = tensor2;
        std::pair<Fr, Fr> upSilu_pair = prove_eleMul(tensor1, tensor2, layer_num, input_tokens, max_embed_dim, eval_point1, eval_point2, upSilu_value);
        done("up * silu");

        size1 = S("Q/gate_out");
        tensor1.get_data(size1, T("Q/gate_out"));
        tensor2.set_size(size1);
        generate_random_eval_points(size1, eval_point1);
        lookup_value = swiglu.prove(tensor1, tensor3, tensor2, eval_point1, hyrax, npoints, commit_time);
        proof = hyrax.open(tensor1, eval_point1, c, size1, max_embed_dim);
        Fr gate_out_value = proof.result;
        proof = hyrax.open(tensor3, eval_point1, c, size1, max_embed_dim);
        require(lookup_value == gate_out_value + proof.result * swiglu.r, "SiLU mapping lookup disagrees with the openings");
        done("SiLU mapping lookup");

        lookup_value = remainder("R/up_out", rs, eval_point2, npoints, max_embed_dim);
        Fr up_out_value = upSilu_pair.first * Fr((long)SCALE1) + lookup_value;
        done("up_out remainder");

        std::pair<Fr, Fr> up_pair = weight_matmul("Q/normOutSecond", "W/up", &tmp_tensor, input_tokens, max_embed_dim, dim, eval_point2, eval_point3, up_out_value);
        const Fr norm_second_out_value1 = up_pair.first;
        done("up projection");

        lookup_value = remainder("R/gate_out", swiglu_rs, eval_point1, npoints, max_embed_dim);
        gate_out_value = gate_out_value * Fr((long)SCALE2) + lookup_value;
        done("gate_out remainder");

        {
            const uint sw = S("W/gate");
            tensor3 = tmp_tensor;
            generate_random_eval_points((size_t)dim * layer_num, eval_point3);
            tensor2.get_data(sw, T("W/gate"));
            tensor1.set_size(sw);
            tensor1 = tensor2;
            tensor3.set_size(S("Q/normOutSecond"));
            std::pair<Fr, Fr> gate_pair = prove_matmul(tensor3, tensor2, layer_num, input_tokens, max_embed_dim, dim, eval_point1, eval_point3, gate_out_value);
            ReassembleVectors(eval_point1, eval_point3, Log2(input_tokens), Log2(dim), Log2(max_embed_dim));
            proof = hyrax.open(tensor1, eval_point3, c, sw, dim);
            require(proof.result == gate_pair.second, "weight opening disagrees with the sumcheck of W/gate");
            const Fr norm_second_out_value2 = gate_pair.first;
            done("gate projection");

            generate_random_eval_points((size_t)dim * layer_num * input_tokens, eval_point3);
            Fr normSecondOut_value = combine_claims(tmp_tensor, {norm_second_out_value1, norm_second_out_value2}, {eval_point2, eval_point1},
                                                    eval_point3, dim * layer_num * input_tokens);
            done("two claims on normOutSecond");

            // ---- second RMSNorm (test/llm.cu:246-297)
            lookup_value = remainder("R/normOutSecond", rs, eval_point3, dim, dim);
            normSecondOut_value = normSecondOut_value * Fr((long)SCALE1) + lookup_value;
            done("normOutSecond remainder");

            size1 = S("Q/skip");
            size2 = S("Q/rmswSecond");
            tensor1.get_data(size1, T("Q/skip"));
            tensor2.get_data(size2, T("Q/rmswSecond"));
            tmp_tensor = tensor1;
            generate_random_eval_points(size1, eval_point1);
            tensor3.set_size(size2);
            tensor3 = tensor2;
            std::pair<Fr, Fr> norm_pair = prove_eleMul(tensor1, tensor2, layer_num, input_tokens, dim, eval_point3, eval_point1, normSecondOut_value);
            done("skip * rmsw");

            lookup_value = remainder("R/rmswSecond", rs, eval_point1, dim, dim);
            Fr rmsw_value = norm_pair.second * Fr((long)SCALE1) + lookup_value;
            done("rmswSecond remainder");

            size1 = S("Q/rmsSecond");
            size2 = S("W/NormSecond");
            generate_random_eval_points(layer_num, eval_point3);
            eval_point2 = eval_point1;
            tensor3.get_data(size1, T("Q/rmsSecond"));
            tensor2.get_data(size2, T("W/NormSecond"));
            tensor1.set_size(size2);
            tensor1 = tensor2;
            std::pair<Fr, Fr> rmsw_pair = prove_matmul(tensor3, tensor2, layer_num, input_tokens, dim, 1, eval_point2, eval_point3, rmsw_value);
            ReassembleVectors(eval_point2, eval_point3, Log2(input_tokens), Log2(1), Log2(dim));
            proof = hyrax.open(tensor1, eval_point3, c, size2, dim / com_scale);
            require(proof.result == rmsw_pair.second, "norm weight opening disagrees");
            tensor1.get_data(size1, T("Q/rmsSecond"));
            proof = hyrax.open(tensor1, eval_point2, c, size1, input_tokens / com_scale);
            require(proof.result == rmsw_pair.first, "rms opening disagrees");
            done("rms (x) norm weight");

            generate_random_eval_points((size_t)dim * layer_num * input_tokens, eval_point2);
            skip_value = combine_claims(tmp_tensor, {skip_value, norm_pair.first}, {skip_eval_point, eval_point1}, eval_point2,
                                        dim * layer_num * input_tokens);
            done("two claims on skip");
        }

        // ======================= attention (test/llm.cu:301-611) =======================
        size1 = S("Q/input");
        tensor1.get_data(size1, T("Q/input"));
        const Fr input_value = hyrax.open(tensor1, eval_point2, c, size1, size1 / layer_num / input_tokens).result;
        Fr atten_out_value = skip_value - input_value;
        done("skip = input + atten_out");

        lookup_value = remainder("R/atten_out", rs, eval_point2, dim, dim);
        atten_out_value = atten_out_value * Fr((long)SCALE1) + lookup_value;
        done("atten_out remainder");

        std::pair<Fr, Fr> O_pair = weight_matmul("Q/qkv", "W/O", nullptr, input_tokens, dim, dim, eval_point2, eval_point3, atten_out_value);
        done("output projection");

        lookup_value = remainder("R/qkv", rs, eval_point2, input_tokens, dim);
        Fr qkv_out_value = O_pair.first * Fr((long)SCALE1) + lookup_value;
        done("qkv remainder");

        // softmax . V: the left matrix is opened, the right one (xv, kept transposed) is proved below
        size1 = S("Q/softmax_output");
        size2 = S("Q/xv");
        generate_random_eval_points((size_t)layer_num * input_tokens, eval_point3);
        tensor3.get_data(size1, T("Q/softmax_output"));
        tensor2.get_data(size2, T("Q/xv"));
        tensor1.set_size(size1);
        tensor1 = tensor3;
        std::pair<Fr, Fr> qkv_pair = prove_matmul(tensor3, tensor2, layer_num, input_tokens, dim, input_tokens, eval_point2, eval_point3, qkv_out_value);
        ReassembleVectors(eval_point2, eval_point3, Log2(input_tokens), Log2(input_tokens), Log2(dim));
        skip_eval_point = eval_point3;
        tensor2.set_size(size1);
        tensor2 = tensor1;
        proof = hyrax.open(tensor1, eval_point2, c, size1, input_tokens);
        require(proof.result == qkv_pair.first, "softmax opening disagrees with the sumcheck of softmax . V");
        done("softmax . V");

        // the softmax relation 2*S*exp - sum*(2*out - 1), rebuilt from exp_output and softmax_output
        // with tensor arithmetic as the reference does (test/llm.cu:381-391)
        size1 = S("Q/exp_output");
        tensor1.get_data(size1, T("Q/exp_output"));
        tensor3.set_size(size1);
        tensor3 = tensor1;
        tensor3 *= (SCALE1 * 2);
        tensor2 *= 2u;
        tensor2 += -1;
        {
            FrTensor row_sums = tensor1.sum(size1, input_tokens);
            tensor2 *= row_sums;
        }
        tensor3 -= tensor2;
        {
            FrTensor query(size1, T("Q/softmax_lookup_query"));
            FrTensor diff(tensor3);
            diff -= query;
            std::vector<Fr> probe = random_vec(Log2(size1));
            require(diff(probe) == Fr::zero(), "the rebuilt softmax relation differs from the generator's lookup query");
        }
        // The reference range-checks this tensor against [0, 2^16) (test/llm.cu:58,392).  The relation
        // only bounds it by twice the row's sum of exponentials, so the check is run when the data
        // allows it and reported otherwise.
        {
            std::vector<int> q(size1);
            require(grape_memcpy_d2h(q.data(), lw.tensor("Q/softmax_lookup_query"), sizeof(int) * (size_t)size1, nullptr) == 0, "d2h");
            int lo = q[0], hi = q[0];
            for (int v : q) { lo = v < lo ? v : lo; hi = v > hi ? v : hi; }
            require(lo >= 0, "negative softmax relation value");
            tensor2.set_size(size1);
            generate_random_eval_points(size1, eval_point1);
            if (hi < (1 << 16)) {
                softmax_range_relation.prove(tensor3, tensor2, eval_point1, hyrax, input_tokens, commit_time);
                done("softmax relation range");
            } else {
                std::printf("  softmax relation values reach %d (rows sum far above one table entry): range lookup over [0, 2^16) not applicable\n", hi);
            }
        }
        tensor3.set_size(size1);
        tensor3 = tensor1;
        hyrax.open(tensor1, eval_point1, c, size1, input_tokens);
        done("exp_output opening");

        size1 = S("Q/exp_input");
        tensor1.get_data(size1, T("Q/exp_input"));
        tensor2.set_size(size1);
        generate_random_eval_points(size1, eval_point1);
        lookup_value = exp.prove(tensor1, tensor3, tensor2, eval_point1, hyrax, input_tokens, commit_time);
        proof = hyrax.open(tensor1, eval_point1, c, size1, input_tokens);
        const Fr exp_in_value = proof.result;
        proof = hyrax.open(tensor3, eval_point1, c, size1, input_tokens);
        require(lookup_value == exp_in_value + proof.result * exp.r, "exp mapping lookup disagrees with the openings");
        done("exp mapping lookup");

        size1 = S("Q/scores");
        tensor1.get_data(size1, T("Q/scores"));
        tensor2.get_data(S("R/scores"), T("R/scores"));
        Fr score_value = tensor1(eval_point1);
        tensor3.set_size(size1);
        tensor3 = tensor2;
        proof = hyrax.open(tensor3, eval_point1, c, size1, input_tokens);
        score_value = score_value * Fr((long)(1 << 22)) + proof.result;
        done("scores quotient and remainder");

        generate_random_eval_points((size_t)layer_num * dim, eval_point2);
        tensor1.get_data(S("Q/xq"), T("Q/xq"));
        tensor2.get_data(S("Q/xk"), T("Q/xk"));
        std::pair<Fr, Fr> qk_pair = prove_matmul(tensor1, tensor2, layer_num, input_tokens, input_tokens, dim, eval_point1, eval_point2, score_value);
        ReassembleVectors(eval_point1, eval_point2, Log2(input_tokens), Log2(dim), Log2(input_tokens));
        done("q . k^T");

        lookup_value = remainder("R/xq", rs, eval_point1, dim, dim);
        Fr q_value = qk_pair.first * Fr((long)SCALE1) + lookup_value;
        done("xq remainder");
        std::pair<Fr, Fr> q_pair = weight_matmul("Q/normOutFirst", "W/Q", nullptr, input_tokens, dim, dim, eval_point1, eval_point3, q_value);
        const Fr norm_first_out1 = q_pair.first;
        done("query projection");

        lookup_value = remainder("R/xk", rs, eval_point2, dim, dim);
        Fr k_value = qk_pair.second * Fr((long)SCALE1) + lookup_value;
        done("xk remainder");
        std::vector<Fr> eval_point_k;
        std::pair<Fr, Fr> k_pair = weight_matmul("Q/normOutFirst", "W/K", nullptr, input_tokens, dim, dim, eval_point2, eval_point_k, k_value);
        const Fr norm_first_out2 = k_pair.first;
        done("key projection");

        lookup_value = remainder("R/xv", rs, skip_eval_point, dim, dim);
        Fr v_value = qkv_pair.second * Fr((long)SCALE1) + lookup_value;
        done("xv remainder");
        {
            // (A B)^T = B^T A^T: the value projection is proved on the transposed product (test/llm.cu:524-535)
            size1 = S("Q/normOutFirst");
            size2 = S("W/V");
            generate_random_eval_points((size_t)layer_num * dim, eval_point3);
            tensor3.get_data(size1, T("Q/normOutFirst"));
            tensor2.get_data(size2, T("W/V"));
            tensor1.set_size(size2);
            tensor1 = tensor2;
            std::pair<Fr, Fr> v_pair = prove_matmul(tensor2, tensor3, layer_num, dim, input_tokens, dim, skip_eval_point, eval_point3, v_value);
            ReassembleVectors(skip_eval_point, eval_point3, Log2(dim), Log2(dim), Log2(input_tokens));
            proof = hyrax.open(tensor1, skip_eval_point, c, size2, dim);
            require(proof.result == v_pair.first, "weight opening disagrees with the sumcheck of W/V");
            const Fr norm_first_out3 = v_pair.second;
            done("value projection (transposed)");

            tensor1.get_data(size1, T("Q/normOutFirst"));
            generate_random_eval_points(size1, skip_eval_point);
            Fr normFirstOut_value = combine_claims(tensor1, {norm_first_out1, norm_first_out2, norm_first_out3},
                                                   {eval_point1, eval_point2, eval_point3}, skip_eval_point, size1);
            done("three claims on normOutFirst");

            // ---- first RMSNorm (test/llm.cu:548-598)
            eval_point3 = skip_eval_point;
            lookup_value = remainder("R/normOutFirst", rs, eval_point3, dim, dim);
            normFirstOut_value = normFirstOut_value * Fr((long)SCALE1) + lookup_value;
            done("normOutFirst remainder");

            size1 = S("Q/input");
            size2 = S("Q/rmswFirst");
            tensor1.get_data(size1, T("Q/input"));
            tensor2.get_data(size2, T("Q/rmswFirst"));
            tmp_tensor = tensor1;
            generate_random_eval_points(size1, eval_point1);
            tensor3.set_size(size2);
            tensor3 = tensor2;
            std::pair<Fr, Fr> norm_pair = prove_eleMul(tensor1, tensor2, layer_num, input_tokens, dim, eval_point3, eval_point1, normFirstOut_value);
            done("input * rmsw");

            lookup_value = remainder("R/rmswFirst", rs, eval_point1, dim, dim);
            Fr rmsw_value = norm_pair.second * Fr((long)SCALE1) + lookup_value;
            done("rmswFirst remainder");

            size1 = S("Q/rmsFirst");
            size2 = S("W/NormFirst");
            generate_random_eval_points(layer_num, eval_point3);
            eval_point2 = eval_point1;
            tensor3.get_data(size1, T("Q/rmsFirst"));
            tensor2.get_data(size2, T("W/NormFirst"));
            tensor1.set_size(size2);
            tensor1 = tensor2;
            std::pair<Fr, Fr> rmsw_pair = prove_matmul(tensor3, tensor2, layer_num, input_tokens, dim, 1, eval_point2, eval_point3, rmsw_value);
            ReassembleVectors(eval_point2, eval_point3, Log2(input_tokens), Log2(1), Log2(dim));
            proof = hyrax.open(tensor1, eval_point3, c, size2, dim / com_scale);
            require(proof.result == rmsw_pair.second, "norm weight opening disagrees");
            tensor1.get_data(size1, T("Q/rmsFirst"));
            proof = hyrax.open(tensor1, eval_point2, c, size1, input_tokens / com_scale);
            require(proof.result == rmsw_pair.first, "rms opening disagrees");
            done("rms (x) norm weight, first");

            const Fr block_input_value = hyrax.open(tmp_tensor, eval_point1, c, layer_num * input_tokens * dim, dim).result;
            require(block_input_value == norm_pair.first, "the block input's opening disagrees with the last claim on it");
            done("block input opening");
        }

        std::printf("layer_flow OK: %d steps, %.1f s, of which %.1f s commitments inside lookups\n", steps,
                    std::chrono::duration<double>(std::chrono::steady_clock::now() - t_start).count(), commit_time);
        return 0;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "%s\n", e.what());
        return 1;
    }
}
