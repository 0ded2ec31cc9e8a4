// SofieFunctor: wraps the infer() of a generated Session in a callable with one float argument per input value
// and a leading slot number, the signature RDataFrame::DefineSlot expects. Same template names, constructor
// arguments and behaviour as the reference's SOFIEHelpers.hxx:11-70 (one Session per slot, slot 0 only when
// nslots is 0, the first output value returned as double). Every Session owns its own device context and
// stream, so slots used from different threads run independently on the GPU.
#ifndef SOFIE_SOFIE_HELPERS
#define SOFIE_SOFIE_HELPERS

#include <string>
#include <type_traits>
#include <utility>
#include <vector>

template <typename I, typename F, typename T>
class SofieFunctorHelper;

template <std::size_t... N, typename Session_t, typename T>
class SofieFunctorHelper<std::index_sequence<N...>, Session_t, T> {
   template <std::size_t Idx>
   using AlwaysT = T;   // N arguments, all of type T

   std::vector<std::vector<T>> fInput;
   std::vector<Session_t> fSessions;

public:
   SofieFunctorHelper(unsigned int nslots = 0, const std::string &filename = "") : fInput(1)
   {
      if (nslots < 1) nslots = 1;
      fInput.resize(nslots);
      fSessions.reserve(nslots);
      for (unsigned int i = 0; i < nslots; i++) {
         if (filename.empty()) fSessions.emplace_back();
         else fSessions.emplace_back(filename);
      }
   }

   double operator()(unsigned slot, AlwaysT<N>... args)
   {
      fInput[slot] = {args...};
      auto y = fSessions[slot].infer(fInput[slot].data());
      return y[0];
   }
};

template <std::size_t N, typename Session_t>
auto SofieFunctor(unsigned int nslots = 0, const std::string &weightsFile = "")
   -> SofieFunctorHelper<std::make_index_sequence<N>, Session_t, float>
{
   return SofieFunctorHelper<std::make_index_sequence<N>, Session_t, float>(nslots, weightsFile);
}

#endif
