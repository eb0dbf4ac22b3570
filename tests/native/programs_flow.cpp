// The reference's six single-protocol test programs (test/matmul.cu, test/eleWiseMul.cu,
// test/combine_value.cu, test/tlookupTest.cu, test/tlookupMapTest.cu, test/HyraxTest.cu), each as one function that keeps
// the program's sequence of calls, run on files in the reference's layouts: the functions read
// points.bin / cpu_points.bin, table/*.bin and {W,Q,R}/<name>-0.bin with loadbin / load_data as the
// programs do.  Differences, all forced: the files hold one block instead of four (the programs'
// `size /= (4 / layer_num)` becomes layer_num = 1 on a one-block file), the direct launches of the
// reference's int_to_fr kernel are FrTensor::get_data (the same conversion), and the widths are a
// small model's (dim 256, feed-forward 1024, 1024 tokens, 1024 x 16 generators; powers of two,
// because the reference hard-codes its 11008 -> 16384 padding).  The programs' CPU_TIMER_* /
// CUDA_TIMER_* / CUDA_DEBUG macros come from ioutils.hpp.  Where a reference program ends
// without looking at its result, the function checks the result against a direct evaluation.
//
// Arguments: working directory (default /tmp/grape_programs_flow).  Prints "programs_flow OK" when
// every check holds.
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <stdexcept>
#include <string>
#include <vector>
#include "artefacts.hpp"
#include "../../grape_amd/host/fr_tensor.hpp"
#include "../../grape_amd/host/hyrax.hpp"
#include "../../grape_amd/host/prove.hpp"
#include "../../grape_amd/host/tlookup.hpp"

static void require(bool ok, const std::string& what) {
    if (!ok) throw std::runtime_error("programs_flow: " + what);
}

static const uint SCALE = 1u << 16;
static const artefacts::Shape kShape = {1024, 256, 1024, 1024, 16};

static fr_t* to_device(const std::vector<Fr>& u) {
    fr_t* d = nullptr;
    require(grape_malloc((void**)&d, sizeof(fr_t) * u.size()) == 0, "grape_malloc");
    require(grape_memcpy_h2d(d, u.data(), sizeof(fr_t) * u.size(), nullptr) == 0, "h2d");
    return d;
}

static Fr first_element(const FrTensor& t) {
    Fr x;
    require(grape_memcpy_d2h(&x, t.gpu_data, sizeof(Fr), nullptr) == 0, "d2h");
    return x;
}

struct Parameters {
    affine_t* points = nullptr;
    std::vector<bn128> cpu_points;
};

// the opening lines of test/tlookupTest.cu:27-33 (and of every program that commits)
static Parameters load_parameters(const std::string& data, uint npoints, uint com_scale) {
    const size_t W = 1 << 8;
    Parameters p;
    require(grape_malloc((void**)&p.points, (size_t)npoints * com_scale * sizeof(affine_t) * W) == 0, "grape_malloc");
    loadbin(data + "/points.bin", p.points, (size_t)npoints * com_scale * sizeof(affine_t) * W);
    p.cpu_points.resize((size_t)npoints * com_scale);
    loadbin(data + "/cpu_points.bin", p.cpu_points.data(), (size_t)npoints * com_scale * sizeof(bn128), false);
    return p;
}

// test/matmul.cu:17-113
static void program_matmul(const std::string& data, uint layer_num) {
    int *up_data = nullptr, *x_data = nullptr, *y_data = nullptr, *y_rem_data = nullptr;
    const uint up_size = load_data(data + "/W/up-0.bin", &up_data);
    const uint x_size = load_data(data + "/Q/ffn_input-0.bin", &x_data);
    const uint y_size = load_data(data + "/Q/up_out-0.bin", &y_data);
    const uint y_rem_size = load_data(data + "/R/up_out-0.bin", &y_rem_data);
    require(up_size && x_size && y_size && y_rem_size == y_size, "matmul: input files");

    std::vector<Fr> u(Log2(y_size));
    long tmp = x_size;
    tmp = (tmp * up_size) / y_size / layer_num;
    const uint same_size = (uint)std::sqrt((double)tmp);
    std::vector<Fr> v(Log2(same_size * layer_num));
    for (auto& e : u) e = Fr::random_element();
    for (auto& e : v) e = Fr::random_element();
    fr_t* U = to_device(u);

    FrTensor up(up_size), y_rem(y_rem_size), x(x_size), y(y_size);
    up.get_data(up_size, up_data);
    y.get_data(y_size, y_data);
    x.get_data(x_size, x_data);
    y_rem.get_data(y_rem_size, y_rem_data);
    FrTensor x_kept(x), up_kept(up);
    y *= SCALE;
    y += y_rem;
    const uint y_dim2 = up_size / same_size / layer_num;
    y.partial_eval(y_size, U, y_size / y_dim2, Log2(y_dim2), y_dim2);
    y.partial_eval(y_dim2, U, y_dim2, 0, 1);
    Fr claim = first_element(y);
    const uint rows = y.size / layer_num / y_dim2;
    std::pair<Fr, Fr> pr = prove_matmul(x, up, layer_num, rows, y_dim2, same_size, u, v, claim);

    // not in the reference program: the two returned values are the operands at the reassembled points
    ReassembleVectors(u, v, Log2(rows), Log2(same_size), Log2(y_dim2));
    require(x_kept(u) == pr.first, "matmul: activation value");
    require(up_kept(v) == pr.second, "matmul: weight value");
    for (void* p : {(void*)up_data, (void*)x_data, (void*)y_data, (void*)y_rem_data, (void*)U}) grape_free(p);
}

// test/eleWiseMul.cu:18-101
static void program_eleWiseMul(const std::string& data, uint layer_num, uint tokens, uint second_size) {
    int *up_out_data = nullptr, *silu_out_data = nullptr, *upSilu_data = nullptr, *upSilu_rem_data = nullptr;
    const uint up_out_size = load_data(data + "/Q/up_out-0.bin", &up_out_data);
    const uint silu_out_size = load_data(data + "/Q/silu_out-0.bin", &silu_out_data);
    const uint upSilu_size = load_data(data + "/Q/upSilu-0.bin", &upSilu_data);
    const uint upSilu_rem_size = load_data(data + "/R/upSilu-0.bin", &upSilu_rem_data);
    require(up_out_size && up_out_size == silu_out_size && upSilu_size == up_out_size && upSilu_rem_size == up_out_size, "eleWiseMul: input files");

    FrTensor up_out(up_out_size, up_out_data), upSilu_rem(upSilu_rem_size, upSilu_rem_data);
    FrTensor silu_out(silu_out_size, silu_out_data), upSilu(upSilu_size, upSilu_data);
    FrTensor up_out_kept(up_out), silu_out_kept(silu_out);
    upSilu *= SCALE;
    upSilu += upSilu_rem;

    std::vector<Fr> u(Log2(upSilu_size)), v(Log2(upSilu_size));
    for (auto& e : u) e = Fr::random_element();
    for (auto& e : v) e = Fr::random_element();
    fr_t* U = to_device(u);
    upSilu.partial_eval(upSilu_size, U, upSilu_size / second_size, Log2(second_size), second_size);
    upSilu.partial_eval(second_size, U, second_size, 0, 1);
    Fr claim = first_element(upSilu);
    CPU_TIMER_START(prove_eleMul);
    std::pair<Fr, Fr> pr = prove_eleMul(up_out, silu_out, layer_num, tokens, second_size, u, v, claim);
    CUDA_DEBUG;
    CPU_TIMER_STOP(prove_eleMul);

    // not in the reference program: the returned values are the two factors at v
    require(up_out_kept(v) == pr.first, "eleWiseMul: first factor");
    require(silu_out_kept(v) == pr.second, "eleWiseMul: second factor");
    for (void* p : {(void*)up_out_data, (void*)silu_out_data, (void*)upSilu_data, (void*)upSilu_rem_data, (void*)U}) grape_free(p);
}

// test/combine_value.cu:14-48
static void program_combine_value(const std::string& data) {
    int* tensor = nullptr;
    const uint size = load_data(data + "/Q/ffn_input-0.bin", &tensor);
    require(size != 0, "combine_value: input file");
    FrTensor X(size, tensor);
    auto u1 = random_vec(Log2(size));
    auto u2 = random_vec(Log2(size));
    Fr claim1 = X(u1);
    X.get_data(size, tensor);
    Fr claim2 = X(u2);
    X.get_data(size, tensor);
    auto v1 = random_vec(Log2(size));
    CPU_TIMER_START(combine);
    const Fr merged = combine_claims(X, {claim1, claim2}, {u1, u2}, v1, size);
    CUDA_DEBUG;
    CPU_TIMER_STOP(combine);
    // not in the reference program: the merged claim is the tensor at v1
    X.get_data(size, tensor);
    require(X(v1) == merged, "combine_value: merged claim");
    grape_free(tensor);
}

// test/tlookupTest.cu:19-63
static void program_tlookupTest(const std::string& data, uint layer_num, const artefacts::Shape& sh) {
    const uint lower = -(1 << 15);
    Parameters pp = load_parameters(data, sh.npoints, sh.com_scale);
    Hyrax hyrax(layer_num, sh.npoints, pp.points, pp.cpu_points[0]);
    int* x_data = nullptr;
    const uint x_size = load_data(data + "/R/up_out-0.bin", &x_data);
    require(x_size != 0, "tlookupTest: input file");

    tLookupRange rs((int)lower, SCALE);
    double com_time = 0.0;
    FrTensor x_tensor(layer_num * sh.tokens * sh.hidden), tlookup_A(layer_num * sh.tokens * sh.hidden);
    x_tensor.get_data(x_size, x_data);
    FrTensor kept(x_tensor);
    auto v = random_vec(Log2(x_size));
    CUDA_TIMER_START(test);
    const Fr value = rs.prove(x_tensor, tlookup_A, v, hyrax, sh.hidden, com_time);
    CUDA_TIMER_STOP(test);
    // not in the reference program: the returned value is the witness at v
    require(kept(v) == value, "tlookupTest: returned value");

    // and a witness with one element outside [-2^15, 2^15) is refused
    std::vector<int> one = {1 << 15};
    require(grape_memcpy_h2d(x_data + 12345, one.data(), sizeof(int), nullptr) == 0, "h2d");
    x_tensor.get_data(x_size, x_data);
    bool refused = false;
    try {
        rs.prove(x_tensor, tlookup_A, v, hyrax, sh.hidden, com_time);
    } catch (const std::exception&) {
        refused = true;
    }
    require(refused, "tlookupTest: an out-of-range witness was accepted");
    grape_free(x_data);
    grape_free(pp.points);
}

// test/tlookupMapTest.cu:21-70
static void program_tlookupMapTest(const std::string& data, uint layer_num, const artefacts::Shape& sh) {
    const int lower = -(1 << 20) + 1;
    const uint length = 1 << 20;
    Parameters pp = load_parameters(data, sh.npoints, sh.com_scale);
    Hyrax hyrax(layer_num, sh.npoints, pp.points, pp.cpu_points[0]);
    int *in_data = nullptr, *out_data = nullptr;
    const uint in_size = load_data(data + "/Q/exp_input-0.bin", &in_data);
    const uint out_size = load_data(data + "/Q/exp_output-0.bin", &out_data);
    require(in_size != 0 && in_size == out_size, "tlookupMapTest: input files");

    tLookupRangeMapping exp(lower, length, data + "/table/exp-table.bin");
    FrTensor s_in(in_size), s_out(out_size), A(in_size);
    s_in.get_data(in_size, in_data);
    s_out.get_data(out_size, out_data);
    FrTensor in_kept(s_in), out_kept(s_out);
    double com_time = 0;
    auto v = random_vec(Log2(in_size));
    const Fr value = exp.prove(s_in, s_out, A, v, hyrax, sh.tokens, com_time);
    // not in the reference program (test/llm.cu:405-411 does it with openings): value = in(v) + r * out(v)
    require(in_kept(v) + exp.r * out_kept(v) == value, "tlookupMapTest: returned value");

    // and an output that is not the table's image of its input is refused
    std::vector<int> h(1);
    require(grape_memcpy_d2h(h.data(), out_data + 777, sizeof(int), nullptr) == 0, "d2h");
    h[0] += 1;
    require(grape_memcpy_h2d(out_data + 777, h.data(), sizeof(int), nullptr) == 0, "h2d");
    s_in.get_data(in_size, in_data);
    s_out.get_data(out_size, out_data);
    bool refused = false;
    try {
        exp.prove(s_in, s_out, A, v, hyrax, sh.tokens, com_time);
    } catch (const std::exception&) {
        refused = true;
    }
    require(refused, "tlookupMapTest: a pair outside the table was accepted");
    grape_free(in_data);
    grape_free(out_data);
    grape_free(pp.points);
}

// test/HyraxTest.cu:16-131, with the verifier's two equations checked on the host exactly as there
// (host_partial_me over the row commitments, a host-side sum of z_j * G_j, the three-term check
// on the evaluation) instead of through Hyrax::verify
static void program_HyraxTest(const std::string& data, uint layer_num, const artefacts::Shape& sh) {
    const uint N = 64;                                   // 4096 in the reference; rows of N * com_scale
    const uint com_scale = sh.com_scale;
    Parameters pp = load_parameters(data, sh.npoints, com_scale);
    std::vector<bn128>& cpu_points = pp.cpu_points;
    int* tensor = nullptr;
    uint size = N * N * 64;
    generate_data(&tensor, size);
    Hyrax hyrax(layer_num, sh.npoints, pp.points, cpu_points[0]);
    FrTensor fr_tensor(size, tensor);
    FrTensor t1 = FrTensor::random((size / N) * (1 << Log2(N)));
    CPU_TIMER_START(commit);
    pad_int(&tensor, N, 1 << Log2(N), (size / N) * (1 << Log2(N)));
    jacob_t* commitment = hyrax.commit(tensor, (size / N) * (1 << Log2(N)), 1 << Log2(N));
    CUDA_DEBUG;
    CPU_TIMER_STOP(commit);
    CPU_TIMER_START(commit_fr);
    jacob_t* commitment1 = hyrax.commit(t1, (size / N) * (1 << Log2(N)), 1 << Log2(N));
    CUDA_DEBUG;
    CPU_TIMER_STOP(commit_fr);

    std::vector<Fr> eval_point(Log2(size));
    for (uint i = 0; i < Log2(size); i++) eval_point[i] = Fr::random_element();
    Fr c = Fr::random_element();
    CPU_TIMER_START(open);
    auto proof = hyrax.open(fr_tensor, eval_point, c, size, N);
    CUDA_DEBUG;
    CPU_TIMER_STOP(open);

    CPU_TIMER_START(verify);
    std::vector<bn128> host_commitment(size / N / com_scale);
    require(grape_memcpy_d2h(host_commitment.data(), commitment, sizeof(jacob_t) * (size / N / com_scale), nullptr) == 0, "d2h");
    uint start_x = Log2(N * com_scale);
    std::vector<bn128> layer_C_(layer_num);
    for (uint i = 0; i < layer_num; i++) {
        layer_C_[i] = host_partial_me<bn128>(host_commitment.data() + i * (size / com_scale / N / layer_num), size / N / com_scale / layer_num,
                                             eval_point.begin() + start_x, eval_point.end() - Log2(layer_num));
    }
    bn128 C_ = host_partial_me<bn128>(layer_C_.data(), layer_num, eval_point.begin() + Log2(size / layer_num), eval_point.end());
    bn128 commit_z = bn128::zero();
    for (uint j = 0; j < (1u << Log2(N)) * com_scale; j++) commit_z = commit_z + proof.z[j] * cpu_points[j];
    C_ = c * C_;
    C_ = C_ + proof.commit_d;
    require(C_ == commit_z, "HyraxTest: c * C + com(d) != com(z)");
    Fr az = host_partial_me<Fr>(proof.z, (1 << Log2(N)) * com_scale, eval_point.begin(), eval_point.begin() + start_x);
    bn128 left = (c * proof.result) * cpu_points[0] + proof.commit_ad;
    bn128 right = az * cpu_points[0];
    require(left == right, "HyraxTest: c * y * G + com(<a, d>) != <a, z> * G");
    CPU_TIMER_STOP(verify);
    // not in the reference program: the opened value is the tensor at the point
    FrTensor again(size, tensor);
    require(again(eval_point) == proof.result, "HyraxTest: opened value");
    grape_free(tensor);
    grape_free(pp.points);
    grape_free(commitment);
    grape_free(commitment1);
}

int main(int argc, char** argv) {
    const std::string dir = argc > 1 ? argv[1] : "/tmp/grape_programs_flow";
    try {
        auto t0 = std::chrono::steady_clock::now();
        auto lap = [&](const char* what) {
            std::printf("  %-16s ok (%.1f s)\n", what, std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count());
            std::fflush(stdout);
        };
        Fr::seed(4242);
        grape_free(artefacts::write_parameters(dir, kShape));
        artefacts::write_witness(dir, kShape, 17);
        lap("files written");
        program_matmul(dir, 1);
        lap("matmul");
        program_eleWiseMul(dir, 1, kShape.tokens, kShape.hidden);
        lap("eleWiseMul");
        program_combine_value(dir);
        lap("combine_value");
        program_tlookupTest(dir, 1, kShape);
        lap("tlookupTest");
        program_tlookupMapTest(dir, 1, kShape);
        lap("tlookupMapTest");
        program_HyraxTest(dir, 1, kShape);
        lap("HyraxTest");
        std::printf("programs_flow OK: %.1f s\n", std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count());
        return 0;
    } catch (const std::exception& e) {
        std::fprintf(stderr, "%s\n", e.what());
        return 1;
    }
}
