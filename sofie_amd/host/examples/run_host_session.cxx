// Runs a Session generated with Options::kHostCode (code for the host cores: BLAS::sgemm_ / saxpy_ calls and loops).
// Compile with -DSOFIE_MODEL_HEADER='"x.hxx"' -DSOFIE_MODEL_NS=SOFIE_x and, for a model with several inputs,
// -DSOFIE_NUM_INPUTS=n (<input.bin> is then a comma-separated list, one file per input in the order of infer()'s
// arguments). Float tensors in and out, one output.
//   run_host_session <weights.dat> <input.bin> <output.bin> [timed iterations of infer]
// The generated code declares the Fortran BLAS routines it calls and leaves their definition to the program it is
// linked into (the reference links whatever find_package(BLAS) finds). This runner defines sgemm_ and saxpy_ itself
// and forwards them: to the library named by the environment variable SOFIE_BLAS (a path for dlopen; SOFIE_BLAS_PREFIX
// is put in front of the symbol names, e.g. "scipy_" for scipy's OpenBLAS) when it is set, else to the plain loops of
// the column-major definition in this file. The thread count is whatever that library takes from its own
// environment. With iterations the runner prints {"host_ms": median, "best_ms": ..., "blas": ...}.
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <dlfcn.h>
#include <fstream>
#include <iostream>
#include <string>
#include <utility>
#include <vector>

#include SOFIE_MODEL_HEADER

#ifndef SOFIE_NUM_INPUTS
#define SOFIE_NUM_INPUTS 1
#endif

namespace {

using SgemmFn = void (*)(const char *, const char *, const int *, const int *, const int *, const float *, const float *, const int *,
                         const float *, const int *, const float *, float *, const int *);
using SaxpyFn = void (*)(const int *, const float *, const float *, const int *, float *, const int *);

// C := alpha * op(A) * op(B) + beta * C on column-major matrices, sums in increasing k
void LoopSgemm(const char *ta, const char *tb, const int *pm, const int *pn, const int *pk, const float *palpha, const float *A,
               const int *plda, const float *B, const int *pldb, const float *pbeta, float *C, const int *pldc)
{
   const int m = *pm, n = *pn, k = *pk, lda = *plda, ldb = *pldb, ldc = *pldc;
   const bool tra = *ta == 't' || *ta == 'T', trb = *tb == 't' || *tb == 'T';
   const float alpha = *palpha, beta = *pbeta;
   for (int j = 0; j < n; ++j) {
      float *cj = C + static_cast<size_t>(j) * ldc;
      for (int i = 0; i < m; ++i) cj[i] = beta == 0.0f ? 0.0f : beta * cj[i];
      if (!tra) {
         for (int l = 0; l < k; ++l) {
            const float b = alpha * (trb ? B[static_cast<size_t>(l) * ldb + j] : B[static_cast<size_t>(j) * ldb + l]);
            const float *al = A + static_cast<size_t>(l) * lda;
            for (int i = 0; i < m; ++i) cj[i] += b * al[i];
         }
      } else {
         for (int i = 0; i < m; ++i) {
            const float *ai = A + static_cast<size_t>(i) * lda;
            float sum = 0.0f;
            for (int l = 0; l < k; ++l) sum += ai[l] * (trb ? B[static_cast<size_t>(l) * ldb + j] : B[static_cast<size_t>(j) * ldb + l]);
            cj[i] += alpha * sum;
         }
      }
   }
}

void LoopSaxpy(const int *n, const float *alpha, const float *x, const int *incx, float *y, const int *incy)
{
   for (int i = 0; i < *n; ++i) y[static_cast<size_t>(i) * *incy] += *alpha * x[static_cast<size_t>(i) * *incx];
}

struct Blas {
   SgemmFn sgemm = LoopSgemm;
   SaxpyFn saxpy = LoopSaxpy;
   std::string name = "loops of run_host_session.cxx";
   Blas()
   {
      const char *path = std::getenv("SOFIE_BLAS");
      if (!path || !*path) return;
      const char *prefix = std::getenv("SOFIE_BLAS_PREFIX");
      const std::string pre = prefix ? prefix : "";
      void *handle = dlopen(path, RTLD_NOW | RTLD_GLOBAL);
      if (!handle) throw std::runtime_error(std::string("cannot load SOFIE_BLAS: ") + dlerror());
      void *g = dlsym(handle, (pre + "sgemm_").c_str()), *a = dlsym(handle, (pre + "saxpy_").c_str());
      if (!g || !a) throw std::runtime_error(std::string("SOFIE_BLAS has no ") + pre + "sgemm_ / " + pre + "saxpy_");
      sgemm = reinterpret_cast<SgemmFn>(g);
      saxpy = reinterpret_cast<SaxpyFn>(a);
      name = path;
   }
};

Blas &TheBlas()
{
   static Blas blas;
   return blas;
}

std::vector<float> ReadRaw(const std::string &path)
{
   std::ifstream fin(path, std::ios::binary | std::ios::ate);
   if (!fin) throw std::runtime_error("cannot open input file " + path);
   const size_t bytes = fin.tellg();
   fin.seekg(0);
   std::vector<float> x(bytes / sizeof(float));
   fin.read(reinterpret_cast<char *>(x.data()), bytes);
   return x;
}

template <size_t... I>
std::vector<float> InferAll(SOFIE_MODEL_NS::Session &s, std::vector<std::vector<float>> &xs, std::index_sequence<I...>)
{
   return s.infer(xs[I].data()...);
}

}   // namespace

extern "C" void sgemm_(const char *ta, const char *tb, const int *m, const int *n, const int *k, const float *alpha, const float *A,
                       const int *lda, const float *B, const int *ldb, const float *beta, float *C, const int *ldc)
{
   TheBlas().sgemm(ta, tb, m, n, k, alpha, A, lda, B, ldb, beta, C, ldc);
}

extern "C" void saxpy_(const int *n, const float *alpha, const float *x, const int *incx, float *y, const int *incy)
{
   TheBlas().saxpy(n, alpha, x, incx, y, incy);
}

int main(int argc, char **argv)
{
   if (argc < 4) {
      std::cerr << "usage: run_host_session <weights.dat> <input.bin> <output.bin> [iterations]\n";
      return 2;
   }
   try {
      SOFIE_MODEL_NS::Session s(argv[1]);
      std::vector<std::vector<float>> xs;
      {
         const std::string list = argv[2];
         size_t start = 0;
         for (size_t comma; (comma = list.find(',', start)) != std::string::npos; start = comma + 1)
            xs.push_back(ReadRaw(list.substr(start, comma - start)));
         xs.push_back(ReadRaw(list.substr(start)));
         if (xs.size() != SOFIE_NUM_INPUTS) throw std::runtime_error("the model takes " + std::to_string(SOFIE_NUM_INPUTS) + " input files");
      }
      std::vector<float> y = InferAll(s, xs, std::make_index_sequence<SOFIE_NUM_INPUTS>{});
      {
         std::ofstream fout(argv[3], std::ios::binary);
         fout.write(reinterpret_cast<const char *>(y.data()), y.size() * sizeof(float));
         if (!fout) throw std::runtime_error(std::string("cannot write ") + argv[3]);
      }
      const int iters = argc > 4 ? std::atoi(argv[4]) : 0;
      if (iters > 0) {
         std::vector<double> ms;
         for (int i = 0; i < iters; ++i) {
            const auto t0 = std::chrono::steady_clock::now();
            y = InferAll(s, xs, std::make_index_sequence<SOFIE_NUM_INPUTS>{});
            ms.push_back(std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count());
         }
         std::sort(ms.begin(), ms.end());
         std::printf("{\"host_ms\": %.6f, \"best_ms\": %.6f, \"iters\": %d, \"blas\": \"%s\"}\n", ms[ms.size() / 2], ms[0], iters,
                     TheBlas().name.c_str());
      }
   } catch (const std::exception &e) {
      std::cerr << "run_host_session: " << e.what() << "\n";
      return 1;
   }
   return 0;
}
