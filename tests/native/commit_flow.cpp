// The reference's artefact pipeline on this build's host classes, file formats included:
// public parameters as test/ppgen.cu writes them (points.bin, cpu_points.bin), the witness files of
// one transformer block as zzllama/llama/model.py writes them (data/{W,Q,R}/<name>-<l>.bin, here
// from LayerWitness::save), and the commitment files of test/commit.cu (data/com{W,Q,R}/<name>-<l>.bin:
// load_data -> pad_int -> Hyrax::commit -> savebin, with that program's row lengths and
// com_scale = 16).  Then what the reference never checks: commitments read back from the files verify
// openings of the tensors read back from the files.
//
// Arguments: working directory (default /tmp/grape_commit_flow), input_tokens (default 64, a multiple
// of 16).  Prints "commit_flow OK" when every check holds.
#include <sys/stat.h>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>
#include "artefacts.hpp"
#include "../../grape_amd/host/fr_tensor.hpp"
#include "../../grape_amd/host/hyrax.hpp"

static void require(bool ok, const std::string& what) {
    if (!ok) throw std::runtime_error("commit_flow: " + what);
}

struct FileInfo {
    std::string name;
    uint N;
};

int main(int argc, char** argv) {
    const std::string dir = argc > 1 ? argv[1] : "/tmp/grape_commit_flow";
    const uint input_tokens = argc > 2 ? (uint)std::atoi(argv[2]) : 64;
    // test/commit.cu:14-18 with the model scaled down 16 times (4096 -> 256, 11008 -> 688, 16384 -> 1024 points) so that
    // points.bin stays at 400 MB; com_scale and every ratio between row lengths are the reference's
    const uint dim = 256, max_embed_dim = 688, npoints = 1024, com_scale = 16, layer_num = 1;
    try {
        require(input_tokens >= 16 && input_tokens % 16 == 0, "input_tokens must be a multiple of 16");
        auto t0 = std::chrono::steady_clock::now();
        Fr::seed(99);
        const artefacts::Shape shape = {input_tokens, dim, max_embed_dim, npoints, com_scale};

        // ---- test/ppgen.cu: generators, the reference-format table, both files; read back as test/commit.cu:28-32 does
        const size_t ngen = (size_t)npoints * com_scale;
        affine_t* points = artefacts::write_parameters(dir, shape);
        require(grape_memset_zero(points, sizeof(affine_t) * 256 * ngen, nullptr) == 0, "memset");
        loadbin(dir + "/points.bin", points, sizeof(affine_t) * 256 * ngen);
        std::vector<bn128> cpu_points(ngen);
        loadbin(dir + "/cpu_points.bin", cpu_points.data(), ngen * sizeof(bn128), false);
        require(bn128(cpu_points[0]) == Fr(1) * cpu_points[0] && !cpu_points[0].is_zero(), "generator 0 unreadable");
        Hyrax hyrax(layer_num, npoints, points, cpu_points[0]);

        // ---- the witness files of one block
        artefacts::write_witness(dir, shape, 5);
        for (const char* sub : {"/comW", "/comQ", "/comR"}) mkdir((dir + sub).c_str(), 0755);
        std::printf("parameters and witness files written after %.1f s\n", std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count());
        std::fflush(stdout);

        // ---- test/commit.cu:37-183: every file through load_data, pad_int, commit, savebin
        const std::vector<FileInfo> W_files = {{"down-", max_embed_dim}, {"up-", dim}, {"gate-", dim}, {"NormSecond-", dim / com_scale},
                                               {"NormFirst-", dim / com_scale}, {"O-", dim}, {"K-", dim}, {"Q-", dim}, {"V-", dim}};
        const std::vector<FileInfo> R_files = {{"down_out-", dim}, {"up_out-", max_embed_dim}, {"gate_out-", max_embed_dim}, {"upSilu-", max_embed_dim},
                                               {"atten_out-", dim}, {"normOutFirst-", dim}, {"normOutSecond-", dim}, {"qkv-", dim},
                                               {"rmswFirst-", dim}, {"rmswSecond-", dim}, {"scores-", input_tokens}, {"xk-", dim},
                                               {"xv-", dim}, {"xq-", dim}};
        const std::vector<FileInfo> Q_files = {{"exp_input-", input_tokens}, {"exp_output-", input_tokens}, {"softmax_output-", input_tokens},
                                               {"rmsFirst-", input_tokens / com_scale}, {"rmsSecond-", input_tokens / com_scale},
                                               {"gate_out-", max_embed_dim}, {"silu_out-", max_embed_dim}, {"input-", dim}, {"output-", dim}};
        size_t committed = 0;
        int files = 0;
        auto commit_dir = [&](const std::string& sub, const std::vector<FileInfo>& list) {
            for (const FileInfo& f : list) {
                int* tensor = nullptr;
                const uint size = load_data(dir + "/" + sub + "/" + f.name + "0.bin", &tensor);
                const uint N = f.N, pad_N = 1u << Log2(N);
                require(size % N == 0, "file size is no multiple of its row length: " + f.name);
                const uint padded = (size / N) * pad_N;
                pad_int(&tensor, N, pad_N, padded);
                jacob_t* commitment = hyrax.commit(tensor, padded, pad_N);
                // test/commit.cu:66 writes size / N / com_scale points
                savebin(dir + "/com" + sub + "/" + f.name + "0.bin", commitment, sizeof(jacob_t) * (size / N / com_scale));
                require(findsize(dir + "/com" + sub + "/" + f.name + "0.bin") == sizeof(jacob_t) * (size_t)(size / N / com_scale),
                        "commitment file size: " + f.name);
                committed += padded;
                files++;
                grape_free(commitment);
                grape_free(tensor);
            }
        };
        auto t1 = std::chrono::steady_clock::now();
        commit_dir("W", W_files);
        commit_dir("R", R_files);
        commit_dir("Q", Q_files);
        const double commit_s = std::chrono::duration<double>(std::chrono::steady_clock::now() - t1).count();
        std::printf("%d files, %zu padded elements committed in %.2f s (file reads and writes included)\n", files, committed, commit_s);
        std::fflush(stdout);

        // ---- commitments from the files verify openings of the tensors from the files
        const Fr c = Fr::random_element();
        for (const auto& item : {std::make_pair(std::string("W"), FileInfo{"down-", max_embed_dim}), std::make_pair(std::string("R"), FileInfo{"xq-", dim}),
                                 std::make_pair(std::string("Q"), FileInfo{"softmax_output-", input_tokens})}) {
            int* tensor = nullptr;
            const uint size = load_data(dir + "/" + item.first + "/" + item.second.name + "0.bin", &tensor);
            const uint N = item.second.N, pad_N = 1u << Log2(N), padded = (size / N) * pad_N;
            pad_int(&tensor, N, pad_N, padded);
            const uint rows = padded / pad_N / com_scale;
            require(rows == size / N / com_scale, "row count");
            jacob_t* commitment = nullptr;
            require(grape_malloc((void**)&commitment, sizeof(jacob_t) * rows) == 0, "grape_malloc");
            loadbin(dir + "/com" + item.first + "/" + item.second.name + "0.bin", commitment, sizeof(jacob_t) * rows);
            FrTensor t(padded, tensor), t2(padded, tensor);
            std::vector<Fr> point = random_vec(Log2(padded));
            Hyrax_proof proof = hyrax.open(t, point, c, padded, pad_N);
            require(hyrax.verify(proof, commitment, point, c, padded, pad_N), "the stored commitment does not verify the opening of " + item.second.name);
            require(proof.result == t2(point), "opened value differs from the multilinear extension of " + item.second.name);
            // a tampered commitment file must not verify
            bn128 first;
            require(grape_memcpy_d2h(&first, commitment, sizeof(jacob_t), nullptr) == 0, "d2h");
            bn128 bad = first + cpu_points[1];
            require(grape_memcpy_h2d(commitment, &bad, sizeof(jacob_t), nullptr) == 0, "h2d");
            FrTensor t3(padded, tensor);
            Hyrax_proof proof2 = hyrax.open(t3, point, c, padded, pad_N);
            require(!hyrax.verify(proof2, commitment, point, c, padded, pad_N), "a tampered commitment verified");
            grape_free(commitment);
            grape_free(tensor);
        }
        std::printf("commit_flow OK: %.1f s\n", std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count());
        return 0;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "%s\n", e.what());
        return 1;
    }
}
