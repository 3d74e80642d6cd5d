// Stand-alone C++ host for the encoder: reads a problem file, runs et::Encoder (include/et.hpp) and writes the result.
// The GPU tests use it to show that the C ABI gives the same bits from C++ as from the Python mirror.
//
//   et_encoder_example <problem.bin> <output.bin>
//
// problem.bin (little endian): int32 dtype (0 fp32, 1 fp16), batch, seq_len, head_num, size_per_head, layers;
// then mask int32 [B,S], from_tensor [B,S,H], attr_mask [B,S,S], and per layer the 16 tensors in the order of the
// reference's `weights_value` (python/effective_transformer/__init__.py:55-74), all in dtype.
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../include/et.hpp"

namespace {

std::vector<char> read_exact(FILE* f, size_t bytes) {
  std::vector<char> v(bytes);
  if (bytes && fread(v.data(), 1, bytes, f) != bytes) throw std::runtime_error("problem file too short");
  return v;
}

void* upload(et::DeviceBuffer& buf, const std::vector<char>& host) {
  void* p = buf.reserve(host.size() ? host.size() : 16);
  et::check_hip(hipMemcpy(p, host.data(), host.size(), hipMemcpyHostToDevice), "hipMemcpy");
  return p;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc != 3) {
    fprintf(stderr, "usage: %s problem.bin output.bin\n", argv[0]);
    return 2;
  }
  try {
    FILE* f = fopen(argv[1], "rb");
    if (!f) throw std::runtime_error("cannot open problem file");
    int32_t hdr[6];
    if (fread(hdr, sizeof(int32_t), 6, f) != 6) throw std::runtime_error("problem file too short");
    const et_dtype dtype = hdr[0] == 0 ? ET_FP32 : ET_FP16;
    const int B = hdr[1], S = hdr[2], heads = hdr[3], d = hdr[4], L = hdr[5];
    const size_t e = dtype == ET_FP32 ? 4 : 2, H = (size_t)heads * d, F = 4 * H;
    et::DeviceBuffer mask_d, x_d, attr_d, out_d;
    const void* mask = upload(mask_d, read_exact(f, (size_t)B * S * 4));
    const void* x = upload(x_d, read_exact(f, (size_t)B * S * H * e));
    const void* attr = upload(attr_d, read_exact(f, (size_t)B * S * S * e));
    // slot sizes in elements: q_k,q_b,k_k,k_b,v_k,v_b,ao_k,ao_b,ao_ln_beta,ao_ln_gamma,i_k,i_b,o_k,o_b,o_ln_beta,o_ln_gamma
    const size_t slot[16] = {H * H, H, H * H, H, H * H, H, H * H, H, H, H, H * F, F, F * H, H, H, H};
    std::vector<et::DeviceBuffer> wbuf((size_t)L * 16);
    std::vector<et_layer_weights> layers((size_t)L);
    for (int l = 0; l < L; ++l) {
      const void* p[16];
      for (int s = 0; s < 16; ++s) p[s] = upload(wbuf[(size_t)l * 16 + s], read_exact(f, slot[s] * e));
      et_layer_weights& w = layers[l];
      w.attr_kernel_Q = p[0]; w.attr_bias_Q = p[1]; w.attr_kernel_K = p[2]; w.attr_bias_K = p[3];
      w.attr_kernel_V = p[4]; w.attr_bias_V = p[5]; w.attr_output_kernel = p[6]; w.attr_output_bias = p[7];
      w.attr_output_layernorm_beta = p[8]; w.attr_output_layernorm_gamma = p[9];
      w.inter_kernel = p[10]; w.inter_bias = p[11]; w.output_kernel = p[12]; w.output_bias = p[13];
      w.output_layernorm_beta = p[14]; w.output_layernorm_gamma = p[15];
    }
    fclose(f);
    void* out = out_d.reserve((size_t)B * S * H * e);
    hipStream_t stream;
    et::check_hip(hipStreamCreate(&stream), "hipStreamCreate");
    et::Encoder enc(0, dtype, heads, d, layers);
    const int T = enc.forward(x, (const int32_t*)mask, attr, out, B, S, stream);
    et::check_hip(hipStreamSynchronize(stream), "hipStreamSynchronize");
    std::vector<char> host((size_t)B * S * H * e);
    et::check_hip(hipMemcpy(host.data(), out, host.size(), hipMemcpyDeviceToHost), "hipMemcpy");
    FILE* g = fopen(argv[2], "wb");
    if (!g || fwrite(host.data(), 1, host.size(), g) != host.size()) throw std::runtime_error("cannot write output file");
    fclose(g);
    et::check_hip(hipStreamDestroy(stream), "hipStreamDestroy");
    printf("valid tokens %d of %d\n", T, B * S);
    return 0;
  } catch (const std::exception& ex) {
    fprintf(stderr, "et_encoder_example: %s\n", ex.what());
    return 1;
  }
}
