// Quantised-layer witness generator: every tensor the reference's Python model writes for one
// transformer block (zzllama/llama/model.py:216-257 RMSNorm, :473-590 attention, :634-703
// feed-forward, :760-775 block), computed on the GPU from int32 activations, weights and tables.
// Tensor names are the reference's file names, "<W|Q|R>/<name>" for data/<W|Q|R>/<name>-<g>.bin.
//
// Rules (model.py:22-24, :76-116, :489-491): scales 2^16 / 2^20 (gate) / 2^22 (scores); every
// rescaling is q = floor((y + S/2)/S), r = y - q*S; products are exact 64-bit integers; softmax and
// SiLU go through their tables; one attention head, no rotary embedding, no mask.  The RMS factor
// is float16(1/sqrt(sum(x^2)/(dim*2^32) + eps)) from the exact integer sum of squares in IEEE
// double arithmetic on the host (the reference takes the same quantity in float32 on the GPU; the
// two can differ by one float16 step at a rounding tie - rms is an advice value of the prover).
#pragma once
#include <map>
#include <string>
#include <vector>

typedef unsigned int uint;

class LayerWitness {
public:
    struct Weights {   // device int32, already scaled by 2^16 (model.py:473-476, :637-639, :224)
        const int *Q, *K, *V, *O;            // dim x dim, row = output feature
        const int *gate, *up;                // hidden x dim
        const int* down;                     // dim x hidden
        const int *norm_first, *norm_second; // dim
    };
    struct Tables {    // device int32
        const int* exp;    // 2^20 entries, entry i <-> x = i - (2^20 - 1)   (model.py:565, test/llm.cu:64)
        const int* silu;   // 2^19 entries, entry i <-> x = i - 2^18         (model.py:666, test/llm.cu:63)
    };
    static const int SCALE_BITS = 16, SWIGLU_SCALE_BITS = 20, QK_SCALE_BITS = 22;

    LayerWitness(uint seq_len, uint dim, uint hidden);
    ~LayerWitness();
    LayerWitness(const LayerWitness&) = delete;
    LayerWitness& operator=(const LayerWitness&) = delete;

    // x: device int32 [seq_len x dim] at scale 2^16.  Throws std::runtime_error when a condition the
    // reference asserts fails (table index out of range) or a value leaves its integer type.
    void generate(const int* x, const Weights& w, const Tables& t, double eps = 1e-5);

    std::vector<std::string> names() const;            // every tensor of the layer, weights included (after generate)
    const int* tensor(const std::string& name) const;  // device pointer; throws on an unknown name
    size_t tensor_size(const std::string& name) const; // elements
    // Appends every tensor to <data_dir>/<W|Q|R>/<name>-<group>.bin as raw little-endian int32, the
    // way the reference's save_int does (model.py:46-63); the three directories must exist.
    void save(const std::string& data_dir, uint group) const;

    // The two tables at the scales the model implies (the reference reads them from files that are
    // not in its tree): exp[i] = round(2^16 exp((i - (2^20-1)) / 2^16)),
    // silu[i] = round(2^16 x sigmoid(x)), x = (i - 2^18) / 2^12.
    static std::vector<int> make_exp_table();
    static std::vector<int> make_silu_table();
    // round-to-nearest-even of a double to IEEE float16, returned as a double
    static double to_float16(double x);

    const uint seq_len, dim, hidden;

private:
    struct Slot { int* owned; const int* ptr; size_t size; };
    std::map<std::string, Slot> t_;
    int* own(const std::string& name, size_t size);
    void alias(const std::string& name, const int* p, size_t size);
    void rmsnorm(const int* x, const int* w, const std::string& tag, double eps);
    unsigned long long* d_sumsq_;
};
