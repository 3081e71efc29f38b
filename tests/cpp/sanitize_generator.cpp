// Host-only driver for runs of the library's host code under AddressSanitizer and UndefinedBehaviorSanitizer
// (built by `make -C acrotensor_amd/csrc asan`; no device is needed: kernels are generated and compiled, never run).
//
//   sanitize_generator spec <file>     the kernels and captures that <file> describes go through the TensorEngine
//                                      (parser, binding, generator, run-time compiler); prints "<name> <fnv1a-64 of
//                                      the emitted source>" per case, so the caller can compare with what the
//                                      ordinary build emits
//   sanitize_generator random <n> <seed>   n seeded random single kernels straight through the generator (no
//                                      compilation), every 10th also through the TensorEngine, plus n / 10 random
//                                      multi-kernel captures (sum-factorised chains of random degree with random
//                                      transient marks); prints a summary line
//
// Spec file, one case after the other:
//   single <name> | <kernel string> | <output dims> ; <input dims> ; ...          (dims separated by commas)
//   chain <name>
//   tensor <tensor name> <dims separated by commas>
//   slice <tensor name> <parent name> <leading indices separated by commas>
//   transient <tensor name>
//   kernel <kernel string> | <output tensor name> <input tensor names ...>
//   end
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <map>
#include <memory>
#include <random>
#include <sstream>
#include <string>
#include <vector>

#include "AcroTensor.hpp"
#include "hip_codegen.hpp"

using namespace acro;

namespace
{

unsigned long long fnv1a(const std::string &s)
{
    unsigned long long h = 1469598103934665603ull;
    for (unsigned char c : s)
    {
        h ^= c;
        h *= 1099511628211ull;
    }
    return h;
}

std::vector<int> dimsOf(const std::string &text)
{
    std::vector<int> dims;
    std::istringstream in(text);
    std::string item;
    while (std::getline(in, item, ','))
    {
        if (!item.empty()) dims.push_back(std::atoi(item.c_str()));
    }
    return dims;
}

std::string trim(const std::string &s)
{
    const size_t a = s.find_first_not_of(" \t"), b = s.find_last_not_of(" \t\r");
    return a == std::string::npos ? std::string() : s.substr(a, b - a + 1);
}

std::vector<std::string> split(const std::string &s, char sep)
{
    std::vector<std::string> parts;
    std::istringstream in(s);
    std::string item;
    while (std::getline(in, item, sep)) parts.push_back(trim(item));
    return parts;
}

int runSpec(const char *path)
{
    std::ifstream in(path);
    if (!in)
    {
        std::printf("cannot read %s\n", path);
        return 2;
    }
    std::string line;
    while (std::getline(in, line))
    {
        line = trim(line);
        if (line.empty() || line[0] == '#') continue;
        if (line.compare(0, 7, "single ") == 0)
        {
            const std::vector<std::string> parts = split(line.substr(7), '|');
            const std::vector<std::string> shapes = split(parts.at(2), ';');
            std::vector<std::unique_ptr<Tensor>> tensors;
            for (const std::string &shape : shapes) tensors.emplace_back(new Tensor(dimsOf(shape)));
            std::vector<Tensor *> inputs;
            for (size_t i = 1; i < tensors.size(); ++i) inputs.push_back(tensors[i].get());
            TensorEngine TE("HIP");
            const std::string src = TE.GetImplementation(parts.at(1), tensors[0].get(), inputs);
            std::printf("%s %016llx\n", parts.at(0).c_str(), fnv1a(src));
        }
        else if (line.compare(0, 6, "chain ") == 0)
        {
            const std::string name = trim(line.substr(6));
            std::map<std::string, std::unique_ptr<Tensor>> tensors;
            std::vector<std::string> order;  // slices are destroyed before their parents
            TensorEngine TE("HIP");
            TE.BeginMultiKernelLaunch();
            while (std::getline(in, line))
            {
                line = trim(line);
                if (line == "end") break;
                std::istringstream words(line);
                std::string what;
                words >> what;
                if (what == "tensor")
                {
                    std::string tname, dims;
                    words >> tname >> dims;
                    tensors[tname].reset(new Tensor(dimsOf(dims)));
                    order.push_back(tname);
                }
                else if (what == "slice")
                {
                    std::string tname, parent, idx;
                    words >> tname >> parent >> idx;
                    tensors[tname].reset(new SliceTensor(*tensors.at(parent), dimsOf(idx)));
                    order.push_back(tname);
                }
                else if (what == "transient")
                {
                    std::string tname;
                    words >> tname;
                    tensors.at(tname)->SetTransient(true);
                }
                else if (what == "kernel")
                {
                    const std::vector<std::string> parts = split(line.substr(7), '|');
                    std::istringstream names(parts.at(1));
                    std::string out, one;
                    names >> out;
                    std::vector<Tensor *> inputs;
                    while (names >> one) inputs.push_back(tensors.at(one).get());
                    TE(parts.at(0), tensors.at(out).get(), inputs);
                }
            }
            const std::string src = TE.EndMultiKernelLaunchGetImplementation();
            std::printf("%s %016llx\n", name.c_str(), fnv1a(src));
            for (size_t i = order.size(); i-- > 0;) tensors.erase(order[i]);
        }
        std::fflush(stdout);
    }
    return 0;
}

struct Random
{
    std::mt19937 rng;
    explicit Random(unsigned seed) : rng(seed) {}
    int operator()(int lo, int hi) { return lo + static_cast<int>(rng() % static_cast<unsigned>(hi - lo + 1)); }
};

// A random kernel "O_<out indices> <op> I0_<...> I1_<...> ...": every contraction index occurs in some input, every
// output index too; extents small except the first output index (the batch) and, now and then, a long contraction.
struct RandomKernel
{
    std::string text;
    std::vector<std::vector<int>> dims;  // output first
};

RandomKernel randomKernel(Random &rnd, int it)
{
    static const char *const names[] = {"e", "i", "j", "k", "l", "m", "n", "q", "r", "s"};
    const int nout = rnd(1, 4), ncon = rnd(0, 3), nidx = nout + ncon;
    std::vector<int> ext(nidx);
    for (int &x : ext) x = rnd(1, 9);
    ext[0] = rnd(1, 3000);
    if (it % 6 == 1 && ncon > 0) ext[nout] = rnd(2048, 6000);                 // split contractions
    if (it % 6 == 2) for (int d = 1; d < nidx; ++d) ext[d] = rnd(10, 70);     // matrices per entry, dense operators
    if (it % 6 == 3 && nout > 1) std::swap(ext[0], ext[nout - 1]);            // the long index last
    const int nin = rnd(1, 4);
    std::vector<std::vector<int>> in(nin);
    for (auto &v : in)
    {
        std::vector<int> pool(nidx);
        for (int d = 0; d < nidx; ++d) pool[d] = d;
        std::shuffle(pool.begin(), pool.end(), rnd.rng);
        v.assign(pool.begin(), pool.begin() + rnd(1, std::min(5, nidx)));
    }
    for (int d = 0; d < nidx; ++d)
    {
        bool used = false;
        for (const auto &v : in)
        {
            for (int x : v) used = used || x == d;
        }
        if (!used) in[rnd(0, nin - 1)].push_back(d);
    }
    // no tensor beyond 2^22 entries: halve the largest extent until every tensor fits
    for (;;)
    {
        double largest = 1.0;
        for (int d = 0; d < nout; ++d) largest *= ext[d];
        for (const auto &v : in)
        {
            double size = 1.0;
            for (int x : v) size *= ext[x];
            largest = std::max(largest, size);
        }
        if (largest <= 4194304.0) break;
        int widest = 0;
        for (int d = 1; d < nidx; ++d)
        {
            if (ext[d] > ext[widest]) widest = d;
        }
        ext[widest] = (ext[widest] + 1) / 2;
    }
    RandomKernel k;
    k.text = "O";
    k.dims.emplace_back();
    for (int d = 0; d < nout; ++d)
    {
        k.text += std::string("_") + names[d];
        k.dims[0].push_back(ext[d]);
    }
    static const char *const ops[] = {" = ", " += ", " -= "};
    k.text += ops[rnd(0, 2)];
    for (int v = 0; v < nin; ++v)
    {
        k.text += (v ? " I" : "I") + std::to_string(v);
        k.dims.emplace_back();
        for (int x : in[v])
        {
            k.text += std::string("_") + names[x];
            k.dims.back().push_back(ext[x]);
        }
    }
    return k;
}

int runRandom(int n, unsigned seed)
{
    Random rnd(seed);
    size_t bytes = 0;
    int fused = 0, through_engine = 0;
    for (int it = 0; it < n; ++it)
    {
        const RandomKernel k = randomKernel(rnd, it);
        std::vector<std::unique_ptr<Tensor>> tensors;
        for (const auto &d : k.dims) tensors.emplace_back(new Tensor(d));
        std::vector<Tensor *> inputs;
        for (size_t i = 1; i < tensors.size(); ++i) inputs.push_back(tensors[i].get());
        try
        {
            TensorKernel parsed(k.text);
            DimensionedKernel bound(&parsed, tensors[0].get(), inputs);
            DimensionedMultiKernel group(&bound);
            HipCodegenOptions options;
            options.transient.assign(group.GetNumUVars(), false);
            options.noalias = rnd(0, 9) != 0;
            const HipKernelPlan plan = GenerateHipKernel(group, options);
            bytes += plan.source.size();
            fused += plan.fusable ? 1 : 0;
            if (it % 10 == 0)
            {
                TensorEngine TE("HIP");
                bytes += TE.GetImplementation(k.text, tensors[0].get(), inputs).size();
                ++through_engine;
            }
        }
        catch (const std::exception &ex)
        {
            std::printf("FAILED %s: %s\n", k.text.c_str(), ex.what());
            return 1;
        }
    }
    // captures: the sum-factorised mass apply at random sizes, random transient marks
    int captures = 0;
    for (int it = 0; it < n / 10; ++it)
    {
        const int P = rnd(2, 6), Q = P + rnd(0, 2), E = rnd(1, 2000);
        Tensor B(Q, P), X(E, P, P, P), D(E, Q, Q, Q), T1(E, Q, P, P), T2(E, Q, Q, P), T3(E, Q, Q, Q), U(E, Q, Q, Q),
            V1(E, P, Q, Q), V2(E, P, P, Q), Y(E, P, P, P);
        for (Tensor *t : {&T1, &T2, &T3, &U, &V1, &V2}) t->SetTransient(rnd(0, 2) != 0);
        try
        {
            TensorEngine TE("HIP");
            TE.BeginMultiKernelLaunch();
            TE("T1_e_q_j_k = B_q_i X_e_i_j_k", T1, B, X);
            TE("T2_e_q_r_k = B_r_j T1_e_q_j_k", T2, B, T1);
            TE("T3_e_q_r_s = B_s_k T2_e_q_r_k", T3, B, T2);
            TE("U_e_q_r_s = D_e_q_r_s T3_e_q_r_s", U, D, T3);
            TE("V1_e_i_r_s = B_q_i U_e_q_r_s", V1, B, U);
            TE("V2_e_i_j_s = B_r_j V1_e_i_r_s", V2, B, V1);
            TE(rnd(0, 1) ? "Y_e_i_j_k = B_s_k V2_e_i_j_s" : "Y_e_i_j_k += B_s_k V2_e_i_j_s", Y, B, V2);
            bytes += TE.EndMultiKernelLaunchGetImplementation().size();
            ++captures;
        }
        catch (const std::exception &ex)
        {
            std::printf("FAILED capture P=%d Q=%d E=%d: %s\n", P, Q, E, ex.what());
            return 1;
        }
    }
    std::printf("random kernels %d (fused %d, through the engine %d), captures %d, %zu bytes of source\n", n, fused,
                through_engine, captures, bytes);
    return 0;
}

}  // namespace

int main(int argc, char **argv)
{
    const std::string mode = argc > 1 ? argv[1] : "";
    if (mode == "spec" && argc > 2) return runSpec(argv[2]);
    if (mode == "random") return runRandom(argc > 2 ? std::atoi(argv[2]) : 300, argc > 3 ? static_cast<unsigned>(std::atoi(argv[3])) : 1u);
    std::printf("usage: sanitize_generator spec <file> | random <n> <seed>\n");
    return 2;
}
