// RSTK checkpoint files (crates/engine/src/checkpoint.rs:1-242; written by
// crates/engine/src/bin/train.rs:609-647):
//   "RSTK", version u32, step u32, dim u32, nlayers u32, vocab u32, seq u32, [activation u32 if version >= 2],
//   then little-endian f32 tensors: embed[V*D], gamma_final[D], and per layer
//   wq wk wv wo w1 w3 w2 gamma1 gamma2.
// The header carries neither heads nor hidden: heads = dim / 128 (hd = 128, MHA) and hidden follows
// from the payload size (checkpoint.rs:101-117, :168-214).
//
// Models the header cannot describe (another head size, grouped KV heads) keep the same file and
// get a side file PATH.shape beside it, one line of text:
//   heads=H kv_heads=K hd=E hidden=F
// The reader takes the shape from the side file when there is one and checks the payload size
// against it; the reference has no such file and reads (or rejects) the main file as before.
//
// Converted checkpoints ("RSTQ", this build's own file; the reference converts nothing ahead of time): the
// weights exactly as the decode library keeps them on the device for one weight format -- so a 4-bit model is
// an eighth of its fp32 file and loads with plain copies:
//   "RSTQ", version u32 (1), step u32, weight format u32 (0 fp32, 1 bf16, 2 e4m3, 3 4-bit), activation u32,
//   dim, hidden, heads, kv_heads, hd, seq, nlayers, vocab (u32 each),
//   gamma_final[D] f32, the embedding, then per layer wqkv, its scales, wo, scales, w13, scales, w2, scales,
//   gamma1[D], gamma2[D]; array sizes are the library's (hipdec_packed_sizes_of).
#pragma once
#include <string>

#include "model.h"

namespace rustane {

struct Checkpoint {
    ModelConfig cfg;
    ModelWeights weights;
    uint32_t step = 0;
};

struct CheckpointShape {
    size_t heads = 0, kv_heads = 0, hd = 0, hidden = 0;
};
// the side file's line; false and a message on anything else
bool parse_checkpoint_shape(const std::string &text, CheckpointShape *out, std::string *err);

// checkpoint.rs:30-166.  Returns false and the reference's message in *err on malformed input.
// shape: the side file's content, or null for a file the header describes.
bool parse_checkpoint(const uint8_t *bytes, size_t len, Checkpoint *out, std::string *err,
                      const CheckpointShape *shape = nullptr);
// checkpoint.rs:25-28 (the file is mapped, not read into a second buffer)
bool load_checkpoint(const std::string &path, Checkpoint *out, std::string *err);
// The converted form: parse (the weights land in out->weights.packed; load_checkpoint tells the two files apart
// by their magic) and write.
bool parse_packed_checkpoint(const uint8_t *bytes, size_t len, Checkpoint *out, std::string *err);
bool write_packed_checkpoint(const std::string &path, const ModelConfig &cfg, const PackedWeights &w, uint32_t step,
                             std::string *err);
// train.rs:609-647: version-2 header and tensor order; a model the header cannot describe
// (hd != 128, kv_heads != heads or dim != heads * 128) also gets the side file
bool write_checkpoint(const std::string &path, const ModelConfig &cfg, const ModelWeights &w, uint32_t step,
                      std::string *err);

}  // namespace rustane
