// Tuned split-KV decode kernel (placeholder selection: nothing covered yet).
#include "ommx_decode_args.h"

namespace ommx {

// Returns 0 when launched, 1 when the shape is not covered by the tuned kernel.
int launch_decode_fast(const DecodeArgs&, int, int, hipStream_t) { return 1; }

}  // namespace ommx
