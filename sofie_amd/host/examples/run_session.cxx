// Runs a generated Session: reads the input tensor from a raw file, calls infer(), writes the output.
// Compile with -DSOFIE_MODEL_HEADER='"x.hxx"' -DSOFIE_MODEL_NS=SOFIE_x -DSOFIE_IN_T=float -DSOFIE_OUT_T=float -DSOFIE_INPUT_MEMBER=fInput_x.
//   run_session <weights.dat> <input.bin> <output.bin> [timed iterations of infer_device]
#include <chrono>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <iostream>
#include <vector>

#include SOFIE_MODEL_HEADER

int main(int argc, char **argv)
{
   if (argc < 4) {
      std::cerr << "usage: run_session <weights.dat> <input.bin> <output.bin> [iterations]\n";
      return 2;
   }
   try {
      SOFIE_MODEL_NS::Session s(argv[1]);
      std::ifstream fin(argv[2], std::ios::binary | std::ios::ate);
      if (!fin) throw std::runtime_error("cannot open input file");
      const size_t bytes = fin.tellg();
      fin.seekg(0);
      std::vector<SOFIE_IN_T> x(bytes / sizeof(SOFIE_IN_T));
      fin.read(reinterpret_cast<char *>(x.data()), bytes);
      std::vector<SOFIE_OUT_T> y = s.infer(x.data());
      std::ofstream fout(argv[3], std::ios::binary);
      fout.write(reinterpret_cast<const char *>(y.data()), y.size() * sizeof(SOFIE_OUT_T));
      const int iters = argc > 4 ? std::atoi(argv[4]) : 0;
      if (iters > 0) {
         // device-resident timing: the input stays in the Session's device buffer
         for (int i = 0; i < 3; ++i) s.infer_device(s.SOFIE_INPUT_MEMBER);
         s.sync();
         float ms = 0;
         sofie_hip_timer_start(s.fCtx);
         for (int i = 0; i < iters; ++i) s.infer_device(s.SOFIE_INPUT_MEMBER);
         sofie_hip_timer_stop(s.fCtx, &ms);
         auto t0 = std::chrono::steady_clock::now();
         for (int i = 0; i < iters; ++i) y = s.infer(x.data());
         const double host_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
         // the same sequence replayed from a HIP graph: outputs must not change, timing of back-to-back replays
         s.use_graph(true);
         std::vector<SOFIE_OUT_T> yg = s.infer(x.data());
         bool same = yg.size() == y.size();
         for (int rep = 0; rep < 3 && same; ++rep) {
            s.infer_device(s.SOFIE_INPUT_MEMBER);   // eager work and a synchronisation between replays
            s.sync();
            yg = s.infer(x.data());
            for (size_t i = 0; i < y.size() && same; ++i) same = std::memcmp(&yg[i], &y[i], sizeof(SOFIE_OUT_T)) == 0;
         }
         s.sync();
         float gms = 0;
         sofie_hip_timer_start(s.fCtx);
         for (int i = 0; i < iters; ++i) s.run_own_input();
         sofie_hip_timer_stop(s.fCtx, &gms);
         std::printf("{\"device_ms\": %.6f, \"host_ms\": %.6f, \"graph_ms\": %.6f, \"graph_matches\": %s, \"iters\": %d}\n", ms / iters,
                     host_ms / iters, gms / iters, same ? "true" : "false", iters);
      }
   } catch (const std::exception &e) {
      std::cerr << "run_session: " << e.what() << "\n";
      return 1;
   }
   return 0;
}
