// SofieFunctor on a generated Session with four input values, the way the reference's RDataFrame tutorial uses it
// (SOFIEHelpers.hxx:56-66): one Session per slot, slots called from their own threads.
//   run_functor <weights.dat> <nslots> <rows.bin (float32, 4 per row)> <out.bin (float64, one per row)>
// Row r is evaluated by slot r % nslots.
#include <cstdio>
#include <fstream>
#include <iostream>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

#include "SOFIE/SOFIEHelpers.hxx"
#include SOFIE_MODEL_HEADER

int main(int argc, char **argv)
{
   if (argc < 5) {
      std::cerr << "usage: run_functor <weights.dat> <nslots> <rows.bin> <out.bin>\n";
      return 2;
   }
   try {
      const unsigned nslots = (unsigned)std::stoul(argv[2]);
      std::ifstream fin(argv[3], std::ios::binary | std::ios::ate);
      if (!fin) throw std::runtime_error(std::string("cannot open ") + argv[3]);
      const size_t bytes = (size_t)fin.tellg();
      fin.seekg(0);
      std::vector<float> rows(bytes / sizeof(float));
      fin.read(reinterpret_cast<char *>(rows.data()), (std::streamsize)bytes);
      const size_t n = rows.size() / 4;
      std::vector<double> out(n);
      auto functor = SofieFunctor<4, SOFIE_MODEL_NS::Session>(nslots, argv[1]);
      std::vector<std::thread> workers;
      const unsigned used = nslots < 1 ? 1 : nslots;
      for (unsigned slot = 0; slot < used; ++slot)
         workers.emplace_back([&, slot]() {
            for (size_t r = slot; r < n; r += used)
               out[r] = functor(slot, rows[4 * r], rows[4 * r + 1], rows[4 * r + 2], rows[4 * r + 3]);
         });
      for (auto &w : workers) w.join();
      std::ofstream fo(argv[4], std::ios::binary);
      fo.write(reinterpret_cast<const char *>(out.data()), (std::streamsize)(n * sizeof(double)));
      std::printf("{\"rows\": %zu, \"slots\": %u}\n", n, used);
   } catch (const std::exception &e) {
      std::cerr << "run_functor: " << e.what() << "\n";
      return 1;
   }
   return 0;
}
