// SofieFunctor<N, Session_t>(nslots, weightsFile): a callable `double(unsigned slot, float x0, ..., float xN-1)`
// over a generated Session, the signature RDataFrame::DefineSlot asks for. The call shape, the meaning of nslots
// (0 or 1: a single Session; otherwise one per slot) and the returned value (the first element of the first
// output) are those of the reference's helper (src/SOFIE_core/inc/SOFIE/SOFIEHelpers.hxx:27-66).
//
// A generated Session here owns a device context, a stream and device buffers, so a slot is a heap object that
// is never copied or moved: copies of the functor (DefineSlot takes it by value) share the slots. Each slot keeps
// its own input row; slots used from different threads run independently on the GPU. A slot number outside the
// range given at construction throws std::out_of_range instead of indexing past the end.
#ifndef SOFIE_SOFIE_HELPERS
#define SOFIE_SOFIE_HELPERS

#include <array>
#include <cstddef>
#include <memory>
#include <string>
#include <utility>
#include <vector>

namespace SOFIE {
namespace Detail {

template <typename Session_t, typename Indices>
class PerSlotCaller;

template <typename Session_t, std::size_t... I>
class PerSlotCaller<Session_t, std::index_sequence<I...>> {
   struct Slot {
      Session_t session;
      std::array<float, sizeof...(I)> row{};
      Slot() : session() {}
      explicit Slot(const std::string &weights) : session(weights) {}
   };
   template <std::size_t>
   using Value = float;   // expands to one float parameter per input value

   std::vector<std::shared_ptr<Slot>> fSlots;

public:
   PerSlotCaller(unsigned int nslots, const std::string &weights)
   {
      const unsigned int count = nslots == 0 ? 1u : nslots;
      fSlots.reserve(count);
      for (unsigned int s = 0; s < count; ++s)
         fSlots.push_back(weights.empty() ? std::make_shared<Slot>() : std::make_shared<Slot>(weights));
   }

   std::size_t slots() const { return fSlots.size(); }

   double operator()(unsigned int slot, Value<I>... values)
   {
      Slot &s = *fSlots.at(slot);
      s.row = {{values...}};
      return static_cast<double>(s.session.infer(s.row.data()).front());
   }
};

}   // namespace Detail
}   // namespace SOFIE

template <std::size_t N, typename Session_t>
SOFIE::Detail::PerSlotCaller<Session_t, std::make_index_sequence<N>> SofieFunctor(unsigned int nslots = 0,
                                                                                 const std::string &weightsFile = "")
{
   return SOFIE::Detail::PerSlotCaller<Session_t, std::make_index_sequence<N>>(nslots, weightsFile);
}

#endif
