// Thin PyTorch extension over the C ABI of libmoe_a2a.so: one torch::Tensor
// wrapper per entry point of include/moe_a2a.h, in the idiom the reference's
// submissions use for their own kernels (wrappers taking torch::Tensor and
// calling data_ptr(), listed in load_inline's `functions=[...]`:
// all2all/hipv8.py:230-252). The reference's wrappers check nothing and launch
// on the null stream; these check device, dtype, contiguity and sizes before
// anything is launched, take the stream to launch on, and turn a nonzero
// status into a Python exception.
//
// The wrappers hold no device code and need no HIP header: they pass pointers
// and sizes on. `shape` is the six ints of struct moe_a2a_shape in field
// order; `stream` is the hipStream_t as an integer
// (torch.cuda.current_stream().cuda_stream).

#include <torch/extension.h>

#include <string>
#include <vector>

#include "moe_a2a.h"

namespace {

moe_a2a_shape shape_of(const std::vector<int64_t>& s) {
  TORCH_CHECK(s.size() == 6,
              "shape: expected [world_size, rank, num_experts, experts_per_token, hidden_dim, max_num_tokens]");
  for (int64_t v : s) TORCH_CHECK(v >= 0 && v <= INT32_MAX, "shape: value out of the int32 range");
  return moe_a2a_shape{(int32_t)s[0], (int32_t)s[1], (int32_t)s[2], (int32_t)s[3], (int32_t)s[4], (int32_t)s[5]};
}

void* stream_of(int64_t stream) { return reinterpret_cast<void*>(static_cast<uintptr_t>(stream)); }

int32_t to_i32(int64_t v, const char* what) {
  TORCH_CHECK(v >= 0 && v <= INT32_MAX, what, ": out of the int32 range");
  return (int32_t)v;
}

// every tensor handed to a kernel: on the GPU, dense, of the expected type and at least `min_numel` long
void need(const torch::Tensor& t, const char* what, c10::ScalarType dt, int64_t min_numel,
          const torch::Tensor* same_device_as = nullptr) {
  TORCH_CHECK(t.is_cuda(), what, ": must be a GPU tensor");
  TORCH_CHECK(t.is_contiguous(), what, ": must be contiguous");
  TORCH_CHECK(t.scalar_type() == dt, what, ": expected ", c10::toString(dt), ", got ", c10::toString(t.scalar_type()));
  TORCH_CHECK(t.numel() >= min_numel, what, ": holds ", t.numel(), " elements, the call needs ", min_numel);
  if (same_device_as) TORCH_CHECK(t.device() == same_device_as->device(), what, ": on another device than the rows");
}

c10::ScalarType rows_type(const torch::Tensor& rows, const char* what) {
  const auto dt = rows.scalar_type();
  TORCH_CHECK(dt == torch::kFloat16 || dt == torch::kBFloat16, what, ": token rows must be float16 or bfloat16");
  return dt;
}

int32_t dtype_code(c10::ScalarType dt) { return dt == torch::kBFloat16 ? MOE_A2A_BF16 : MOE_A2A_F16; }

int32_t* ints(const torch::Tensor& t) { return t.data_ptr<int32_t>(); }

int32_t* ints_or_null(const c10::optional<torch::Tensor>& t) { return t.has_value() ? t->data_ptr<int32_t>() : nullptr; }

void status(int rc, const char* fn) {
  TORCH_CHECK(rc == MOE_A2A_OK, fn, ": status ", rc, " (", moe_a2a_strerror(rc), ")");
}

}  // namespace

std::string a2a_version() { return moe_a2a_version(); }

void a2a_dispatch_send(std::vector<int64_t> shape, torch::Tensor x, torch::Tensor indices, int64_t num_tokens,
                       torch::Tensor send_buf, torch::Tensor send_meta, torch::Tensor send_counts,
                       c10::optional<torch::Tensor> send_slot, int64_t stream) {
  const moe_a2a_shape s = shape_of(shape);
  const int64_t S = num_tokens * s.experts_per_token;
  const auto dt = rows_type(x, "x");
  need(x, "x", dt, num_tokens * s.hidden_dim);
  need(indices, "indices", torch::kInt32, S, &x);
  need(send_buf, "send_buf", dt, S * s.hidden_dim, &x);
  need(send_meta, "send_meta", torch::kInt32, S * MOE_A2A_META_DIM, &x);
  need(send_counts, "send_counts", torch::kInt32, s.world_size, &x);
  if (send_slot.has_value()) need(*send_slot, "send_slot", torch::kInt32, S, &x);
  status(moe_a2a_dispatch_send(&s, x.data_ptr(), ints(indices), to_i32(num_tokens, "num_tokens"),
                               send_buf.data_ptr(), ints(send_meta), ints(send_counts), ints_or_null(send_slot),
                               stream_of(stream)),
         "moe_a2a_dispatch_send");
}

void a2a_plan_send(std::vector<int64_t> shape, torch::Tensor indices, int64_t num_tokens,
                   torch::Tensor rank_counts, torch::Tensor rank_offsets, torch::Tensor expert_counts,
                   torch::Tensor dst_slot, torch::Tensor src_entry, int64_t stream) {
  const moe_a2a_shape s = shape_of(shape);
  const int64_t S = num_tokens * s.experts_per_token;
  need(indices, "indices", torch::kInt32, S);
  need(rank_counts, "rank_counts", torch::kInt32, s.world_size, &indices);
  need(rank_offsets, "rank_offsets", torch::kInt32, s.world_size + 1, &indices);
  need(expert_counts, "expert_counts", torch::kInt32, s.num_experts, &indices);
  need(dst_slot, "dst_slot", torch::kInt32, S, &indices);
  need(src_entry, "src_entry", torch::kInt32, S, &indices);
  status(moe_a2a_plan_send(&s, ints(indices), to_i32(num_tokens, "num_tokens"), ints(rank_counts),
                           ints(rank_offsets), ints(expert_counts), ints(dst_slot), ints(src_entry),
                           stream_of(stream)),
         "moe_a2a_plan_send");
}

void a2a_dispatch_recv(std::vector<int64_t> shape, torch::Tensor recv_buf, torch::Tensor recv_meta,
                       torch::Tensor recv_counts, int64_t rows_hint, torch::Tensor expert_num_tokens,
                       torch::Tensor expert_x, torch::Tensor expert_meta,
                       c10::optional<torch::Tensor> send_back_plan,
                       c10::optional<torch::Tensor> row_position, int64_t stream) {
  const moe_a2a_shape s = shape_of(shape);
  const auto dt = rows_type(recv_buf, "recv_buf");
  const int64_t nle = s.world_size > 0 ? s.num_experts / s.world_size : 0;
  const int64_t padded = nle * s.max_num_tokens * s.world_size;
  need(recv_buf, "recv_buf", dt, 0);
  need(recv_meta, "recv_meta", torch::kInt32, 0, &recv_buf);
  // rows the two receive buffers were allocated with
  const int64_t capacity = std::min(recv_buf.numel() / std::max<int64_t>(s.hidden_dim, 1),
                                    recv_meta.numel() / MOE_A2A_META_DIM);
  need(recv_counts, "recv_counts", torch::kInt32, s.world_size, &recv_buf);
  need(expert_num_tokens, "expert_num_tokens", torch::kInt32, nle, &recv_buf);
  need(expert_x, "expert_x", dt, padded * s.hidden_dim, &recv_buf);
  need(expert_meta, "expert_meta", torch::kInt32, padded * MOE_A2A_META_DIM, &recv_buf);
  if (send_back_plan.has_value())
    need(*send_back_plan, "send_back_plan", torch::kInt32, 2 * (int64_t)s.num_experts, &recv_buf);
  if (row_position.has_value()) {  // long streams: positions from a planning launch
    need(*row_position, "row_position", torch::kInt32, capacity, &recv_buf);
    status(moe_a2a_dispatch_recv_long(&s, recv_buf.data_ptr(), ints(recv_meta), ints(recv_counts),
                                      to_i32(rows_hint, "rows_hint"), to_i32(capacity, "capacity_rows"),
                                      ints(expert_num_tokens), expert_x.data_ptr(), ints(expert_meta),
                                      ints_or_null(send_back_plan), ints(*row_position), stream_of(stream)),
           "moe_a2a_dispatch_recv_long");
    return;
  }
  status(moe_a2a_dispatch_recv(&s, recv_buf.data_ptr(), ints(recv_meta), ints(recv_counts),
                               to_i32(rows_hint, "rows_hint"), to_i32(capacity, "capacity_rows"),
                               ints(expert_num_tokens), expert_x.data_ptr(), ints(expert_meta),
                               ints_or_null(send_back_plan), stream_of(stream)),
         "moe_a2a_dispatch_recv");
}

void a2a_combine_send(std::vector<int64_t> shape, torch::Tensor expert_y, torch::Tensor expert_meta,
                      torch::Tensor expert_num_tokens, int64_t rows_hint, torch::Tensor send_buf,
                      torch::Tensor send_meta, torch::Tensor send_counts,
                      c10::optional<torch::Tensor> send_back_plan, int64_t stream) {
  const moe_a2a_shape s = shape_of(shape);
  const auto dt = rows_type(expert_y, "expert_y");
  const int64_t nle = s.world_size > 0 ? s.num_experts / s.world_size : 0;
  const int64_t padded = nle * s.max_num_tokens * s.world_size;
  need(expert_y, "expert_y", dt, padded * s.hidden_dim);
  need(expert_meta, "expert_meta", torch::kInt32, padded * MOE_A2A_META_DIM, &expert_y);
  need(expert_num_tokens, "expert_num_tokens", torch::kInt32, nle, &expert_y);
  need(send_buf, "send_buf", dt, 0, &expert_y);
  need(send_meta, "send_meta", torch::kInt32, 0, &expert_y);
  const int64_t capacity = std::min(send_buf.numel() / std::max<int64_t>(s.hidden_dim, 1),
                                    send_meta.numel() / MOE_A2A_META_DIM);
  need(send_counts, "send_counts", torch::kInt32, s.world_size, &expert_y);
  if (send_back_plan.has_value())
    need(*send_back_plan, "send_back_plan", torch::kInt32, 2 * (int64_t)s.num_experts, &expert_y);
  status(moe_a2a_combine_send(&s, expert_y.data_ptr(), ints(expert_meta), ints(expert_num_tokens),
                              to_i32(std::min(rows_hint, capacity), "rows_hint"), to_i32(capacity, "capacity_rows"),
                              send_buf.data_ptr(), ints(send_meta), ints(send_counts),
                              ints_or_null(send_back_plan), stream_of(stream)),
         "moe_a2a_combine_send");
}

void a2a_combine_recv(std::vector<int64_t> shape, torch::Tensor recv_buf, torch::Tensor recv_meta,
                      torch::Tensor recv_counts, int64_t rows_hint, torch::Tensor weights, int64_t num_tokens,
                      torch::Tensor out_tokens, bool accumulate, c10::optional<torch::Tensor> entry_row,
                      int64_t stream) {
  const moe_a2a_shape s = shape_of(shape);
  const auto dt = rows_type(out_tokens, "out_tokens");
  need(out_tokens, "out_tokens", dt, num_tokens * s.hidden_dim);
  need(recv_buf, "recv_buf", dt, 0, &out_tokens);
  need(recv_meta, "recv_meta", torch::kInt32, 0, &out_tokens);
  const int64_t capacity = std::min(recv_buf.numel() / std::max<int64_t>(s.hidden_dim, 1),
                                    recv_meta.numel() / MOE_A2A_META_DIM);
  need(recv_counts, "recv_counts", torch::kInt32, s.world_size, &out_tokens);
  need(weights, "weights", torch::kFloat32, num_tokens * s.experts_per_token, &out_tokens);
  if (entry_row.has_value()) {  // long streams: rows looked up in a (token, k) -> row table
    need(*entry_row, "entry_row", torch::kInt32, num_tokens * s.experts_per_token, &out_tokens);
    status(moe_a2a_combine_recv_long(&s, recv_buf.data_ptr(), ints(recv_meta), ints(recv_counts),
                                     to_i32(std::min(rows_hint, capacity), "rows_hint"),
                                     to_i32(capacity, "capacity_rows"), weights.data_ptr<float>(),
                                     to_i32(num_tokens, "num_tokens"), out_tokens.data_ptr(), accumulate ? 1 : 0,
                                     dtype_code(dt), ints(*entry_row), stream_of(stream)),
           "moe_a2a_combine_recv_long");
    return;
  }
  status(moe_a2a_combine_recv(&s, recv_buf.data_ptr(), ints(recv_meta), ints(recv_counts),
                              to_i32(std::min(rows_hint, capacity), "rows_hint"), to_i32(capacity, "capacity_rows"),
                              weights.data_ptr<float>(), to_i32(num_tokens, "num_tokens"), out_tokens.data_ptr(),
                              accumulate ? 1 : 0, dtype_code(dt), stream_of(stream)),
         "moe_a2a_combine_recv");
}

void a2a_expert_scale(std::vector<int64_t> shape, torch::Tensor expert_x, torch::Tensor expert_num_tokens,
                      int64_t rows_hint, torch::Tensor expert_y, int64_t stream) {
  const moe_a2a_shape s = shape_of(shape);
  const auto din = rows_type(expert_x, "expert_x"), dout = rows_type(expert_y, "expert_y");
  const int64_t nle = s.world_size > 0 ? s.num_experts / s.world_size : 0;
  const int64_t padded = nle * s.max_num_tokens * s.world_size;
  need(expert_x, "expert_x", din, padded * s.hidden_dim);
  need(expert_y, "expert_y", dout, padded * s.hidden_dim, &expert_x);
  need(expert_num_tokens, "expert_num_tokens", torch::kInt32, nle, &expert_x);
  status(moe_a2a_expert_scale(&s, expert_x.data_ptr(), ints(expert_num_tokens), to_i32(rows_hint, "rows_hint"),
                              dtype_code(din), dtype_code(dout), expert_y.data_ptr(), stream_of(stream)),
         "moe_a2a_expert_scale");
}

void a2a_expert_gemm(std::vector<int64_t> shape, torch::Tensor expert_x, torch::Tensor expert_num_tokens,
                     int64_t rows_hint, torch::Tensor weights, c10::optional<torch::Tensor> bias,
                     torch::Tensor expert_y, int64_t stream) {
  const moe_a2a_shape s = shape_of(shape);
  const auto dt = rows_type(expert_x, "expert_x");
  const int64_t nle = s.world_size > 0 ? s.num_experts / s.world_size : 0;
  const int64_t padded = nle * s.max_num_tokens * s.world_size;
  TORCH_CHECK(weights.dim() == 3 && weights.size(0) == nle, "weights must be [num_local_experts, out_dim, in_dim]");
  const int64_t out_dim = weights.size(1), in_dim = weights.size(2);
  need(expert_x, "expert_x", dt, padded * in_dim);
  need(expert_y, "expert_y", dt, padded * out_dim, &expert_x);
  need(weights, "weights", dt, nle * out_dim * in_dim, &expert_x);
  need(expert_num_tokens, "expert_num_tokens", torch::kInt32, nle, &expert_x);
  const void* b = nullptr;
  if (bias.has_value()) {
    need(*bias, "bias", dt, nle * out_dim, &expert_x);
    b = bias->data_ptr();
  }
  status(moe_a2a_expert_gemm(&s, expert_x.data_ptr(), ints(expert_num_tokens), to_i32(rows_hint, "rows_hint"),
                             weights.data_ptr(), b, to_i32(in_dim, "in_dim"), to_i32(out_dim, "out_dim"),
                             dtype_code(dt), expert_y.data_ptr(), stream_of(stream)),
         "moe_a2a_expert_gemm");
}

void a2a_linear(torch::Tensor input, torch::Tensor weight, c10::optional<torch::Tensor> bias, torch::Tensor output,
                int64_t stream) {
  const auto dt = rows_type(input, "input");
  TORCH_CHECK(input.dim() == 2 && weight.dim() == 2 && output.dim() == 2, "input, weight and output must be 2-D");
  const int64_t m = input.size(0), k = input.size(1), n = weight.size(0);
  need(input, "input", dt, m * k);
  need(weight, "weight", dt, n * k, &input);
  need(output, "output", dt, m * n, &input);
  TORCH_CHECK(weight.size(1) == k, "weight must be [n, k] with k = input.size(1)");
  TORCH_CHECK(output.size(0) == m && output.size(1) == n, "output must be [m, n]");
  const void* b = nullptr;
  if (bias.has_value()) {
    need(*bias, "bias", dt, n, &input);
    b = bias->data_ptr();
  }
  status(moe_a2a_linear(input.data_ptr(), weight.data_ptr(), b, to_i32(m, "m"), to_i32(n, "n"), to_i32(k, "k"),
                        dtype_code(dt), output.data_ptr(), stream_of(stream)),
         "moe_a2a_linear");
}

void a2a_exchange_local(int64_t world_size, int64_t hidden_dim, torch::Tensor send_buf, torch::Tensor send_meta,
                        torch::Tensor send_counts, int64_t dst_rank, torch::Tensor recv_buf,
                        torch::Tensor recv_meta, torch::Tensor recv_counts, int64_t src_rank, int64_t rows_hint,
                        int64_t stream) {
  const auto dt = rows_type(send_buf, "send_buf");
  need(send_buf, "send_buf", dt, 0);
  need(send_meta, "send_meta", torch::kInt32, 0, &send_buf);
  need(recv_buf, "recv_buf", dt, 0, &send_buf);
  need(recv_meta, "recv_meta", torch::kInt32, 0, &send_buf);
  need(send_counts, "send_counts", torch::kInt32, world_size, &send_buf);
  need(recv_counts, "recv_counts", torch::kInt32, world_size, &send_buf);
  const int64_t h = std::max<int64_t>(hidden_dim, 1);
  const int64_t send_capacity = std::min(send_buf.numel() / h, send_meta.numel() / MOE_A2A_META_DIM);
  const int64_t recv_capacity = std::min(recv_buf.numel() / h, recv_meta.numel() / MOE_A2A_META_DIM);
  status(moe_a2a_exchange_local(to_i32(world_size, "world_size"), to_i32(hidden_dim, "hidden_dim"),
                                send_buf.data_ptr(), ints(send_meta), ints(send_counts),
                                to_i32(dst_rank, "dst_rank"), recv_buf.data_ptr(), ints(recv_meta),
                                ints(recv_counts), to_i32(src_rank, "src_rank"), to_i32(rows_hint, "rows_hint"),
                                to_i32(send_capacity, "send_capacity_rows"),
                                to_i32(recv_capacity, "recv_capacity_rows"), stream_of(stream)),
         "moe_a2a_exchange_local");
}

void a2a_exchange_gather_local(int64_t world_size, int64_t hidden_dim, std::vector<torch::Tensor> send_bufs,
                               std::vector<torch::Tensor> send_metas, std::vector<torch::Tensor> send_counts,
                               int64_t dst_rank, torch::Tensor recv_buf, torch::Tensor recv_meta,
                               torch::Tensor recv_counts, int64_t rows_hint, int64_t stream) {
  TORCH_CHECK(world_size >= 1 && world_size <= 64, "world_size: 1 to 64 source ranks in one launch");
  TORCH_CHECK((int64_t)send_bufs.size() == world_size && (int64_t)send_metas.size() == world_size &&
              (int64_t)send_counts.size() == world_size, "one send_buf, send_meta and send_counts per source rank");
  const auto dt = rows_type(recv_buf, "recv_buf");
  need(recv_buf, "recv_buf", dt, 0);
  need(recv_meta, "recv_meta", torch::kInt32, 0, &recv_buf);
  need(recv_counts, "recv_counts", torch::kInt32, world_size, &recv_buf);
  const int64_t h = std::max<int64_t>(hidden_dim, 1);
  const void* bufs[64];
  const int32_t* metas[64];
  const int32_t* counts[64];
  int64_t send_capacity = INT32_MAX;
  for (int64_t r = 0; r < world_size; ++r) {
    need(send_bufs[r], "send_bufs[r]", dt, 0, &recv_buf);
    need(send_metas[r], "send_metas[r]", torch::kInt32, 0, &recv_buf);
    need(send_counts[r], "send_counts[r]", torch::kInt32, world_size, &recv_buf);
    send_capacity = std::min(send_capacity, std::min(send_bufs[r].numel() / h, send_metas[r].numel() / MOE_A2A_META_DIM));
    bufs[r] = send_bufs[r].data_ptr();
    metas[r] = ints(send_metas[r]);
    counts[r] = ints(send_counts[r]);
  }
  const int64_t recv_capacity = std::min(recv_buf.numel() / h, recv_meta.numel() / MOE_A2A_META_DIM);
  status(moe_a2a_exchange_gather_local(to_i32(world_size, "world_size"), to_i32(hidden_dim, "hidden_dim"), bufs,
                                       metas, counts, to_i32(dst_rank, "dst_rank"), recv_buf.data_ptr(),
                                       ints(recv_meta), ints(recv_counts), to_i32(rows_hint, "rows_hint"),
                                       to_i32(send_capacity, "send_capacity_rows"),
                                       to_i32(recv_capacity, "recv_capacity_rows"), stream_of(stream)),
         "moe_a2a_exchange_gather_local");
}

// ---- the compact expert-major layout: 2-D expert buffers [rows, width], the experts' rows back to back

namespace {
int64_t compact_rows(const torch::Tensor& rows, const char* what) {
  TORCH_CHECK(rows.dim() == 2 && rows.size(0) >= 1, what, ": compact expert buffers are [rows, width] with rows >= 1");
  return rows.size(0);
}
}  // namespace

void a2a_dispatch_recv_compact(std::vector<int64_t> shape, torch::Tensor recv_buf, torch::Tensor recv_meta,
                               torch::Tensor recv_counts, int64_t rows_hint, torch::Tensor expert_num_tokens,
                               torch::Tensor expert_offsets, torch::Tensor expert_x, torch::Tensor expert_meta,
                               c10::optional<torch::Tensor> send_back_plan, int64_t stream) {
  const moe_a2a_shape s = shape_of(shape);
  const auto dt = rows_type(recv_buf, "recv_buf");
  const int64_t nle = s.world_size > 0 ? s.num_experts / s.world_size : 0;
  need(recv_buf, "recv_buf", dt, 0);
  need(recv_meta, "recv_meta", torch::kInt32, 0, &recv_buf);
  const int64_t capacity = std::min(recv_buf.numel() / std::max<int64_t>(s.hidden_dim, 1),
                                    recv_meta.numel() / MOE_A2A_META_DIM);
  const int64_t room = std::min(compact_rows(expert_x, "expert_x"), compact_rows(expert_meta, "expert_meta"));
  need(recv_counts, "recv_counts", torch::kInt32, s.world_size, &recv_buf);
  need(expert_num_tokens, "expert_num_tokens", torch::kInt32, nle, &recv_buf);
  need(expert_offsets, "expert_offsets", torch::kInt32, nle + 1, &recv_buf);
  need(expert_x, "expert_x", dt, room * s.hidden_dim, &recv_buf);
  need(expert_meta, "expert_meta", torch::kInt32, room * MOE_A2A_META_DIM, &recv_buf);
  if (send_back_plan.has_value())
    need(*send_back_plan, "send_back_plan", torch::kInt32, 2 * (int64_t)s.num_experts, &recv_buf);
  status(moe_a2a_dispatch_recv_compact(&s, recv_buf.data_ptr(), ints(recv_meta), ints(recv_counts),
                                       to_i32(std::min(rows_hint, capacity), "rows_hint"),
                                       to_i32(capacity, "capacity_rows"), ints(expert_num_tokens),
                                       ints(expert_offsets), expert_x.data_ptr(), ints(expert_meta),
                                       to_i32(room, "compact_capacity_rows"), ints_or_null(send_back_plan),
                                       stream_of(stream)),
         "moe_a2a_dispatch_recv_compact");
}

void a2a_expert_scale_compact(std::vector<int64_t> shape, torch::Tensor expert_x, torch::Tensor expert_num_tokens,
                              int64_t rows_hint, torch::Tensor expert_y, int64_t stream) {
  const moe_a2a_shape s = shape_of(shape);
  const auto din = rows_type(expert_x, "expert_x"), dout = rows_type(expert_y, "expert_y");
  const int64_t nle = s.world_size > 0 ? s.num_experts / s.world_size : 0;
  const int64_t room = std::min(compact_rows(expert_x, "expert_x"), compact_rows(expert_y, "expert_y"));
  need(expert_x, "expert_x", din, room * s.hidden_dim);
  need(expert_y, "expert_y", dout, room * s.hidden_dim, &expert_x);
  need(expert_num_tokens, "expert_num_tokens", torch::kInt32, nle, &expert_x);
  status(moe_a2a_expert_scale_compact(&s, expert_x.data_ptr(), ints(expert_num_tokens),
                                      to_i32(rows_hint, "rows_hint"), to_i32(room, "compact_capacity_rows"),
                                      dtype_code(din), dtype_code(dout), expert_y.data_ptr(), stream_of(stream)),
         "moe_a2a_expert_scale_compact");
}

void a2a_expert_gemm_compact(std::vector<int64_t> shape, torch::Tensor expert_x, torch::Tensor expert_num_tokens,
                             int64_t rows_hint, torch::Tensor weights, c10::optional<torch::Tensor> bias,
                             torch::Tensor expert_y, int64_t stream) {
  const moe_a2a_shape s = shape_of(shape);
  const auto dt = rows_type(expert_x, "expert_x");
  const int64_t nle = s.world_size > 0 ? s.num_experts / s.world_size : 0;
  TORCH_CHECK(weights.dim() == 3 && weights.size(0) == nle, "weights must be [num_local_experts, out_dim, in_dim]");
  const int64_t out_dim = weights.size(1), in_dim = weights.size(2);
  const int64_t room = std::min(compact_rows(expert_x, "expert_x"), compact_rows(expert_y, "expert_y"));
  need(expert_x, "expert_x", dt, room * in_dim);
  need(expert_y, "expert_y", dt, room * out_dim, &expert_x);
  need(weights, "weights", dt, nle * out_dim * in_dim, &expert_x);
  need(expert_num_tokens, "expert_num_tokens", torch::kInt32, nle, &expert_x);
  const void* b = nullptr;
  if (bias.has_value()) {
    need(*bias, "bias", dt, nle * out_dim, &expert_x);
    b = bias->data_ptr();
  }
  status(moe_a2a_expert_gemm_compact(&s, expert_x.data_ptr(), ints(expert_num_tokens), to_i32(rows_hint, "rows_hint"),
                                     to_i32(room, "compact_capacity_rows"), weights.data_ptr(), b,
                                     to_i32(in_dim, "in_dim"), to_i32(out_dim, "out_dim"), dtype_code(dt),
                                     expert_y.data_ptr(), stream_of(stream)),
         "moe_a2a_expert_gemm_compact");
}

void a2a_combine_send_compact(std::vector<int64_t> shape, torch::Tensor expert_y, torch::Tensor expert_meta,
                              torch::Tensor expert_num_tokens, int64_t rows_hint, torch::Tensor send_buf,
                              torch::Tensor send_meta, torch::Tensor send_counts,
                              c10::optional<torch::Tensor> send_back_plan, int64_t stream) {
  const moe_a2a_shape s = shape_of(shape);
  const auto dt = rows_type(expert_y, "expert_y");
  const int64_t nle = s.world_size > 0 ? s.num_experts / s.world_size : 0;
  const int64_t room = std::min(compact_rows(expert_y, "expert_y"), compact_rows(expert_meta, "expert_meta"));
  need(expert_y, "expert_y", dt, room * s.hidden_dim);
  need(expert_meta, "expert_meta", torch::kInt32, room * MOE_A2A_META_DIM, &expert_y);
  need(expert_num_tokens, "expert_num_tokens", torch::kInt32, nle, &expert_y);
  need(send_buf, "send_buf", dt, 0, &expert_y);
  need(send_meta, "send_meta", torch::kInt32, 0, &expert_y);
  const int64_t capacity = std::min(send_buf.numel() / std::max<int64_t>(s.hidden_dim, 1),
                                    send_meta.numel() / MOE_A2A_META_DIM);
  need(send_counts, "send_counts", torch::kInt32, s.world_size, &expert_y);
  if (send_back_plan.has_value())
    need(*send_back_plan, "send_back_plan", torch::kInt32, 2 * (int64_t)s.num_experts, &expert_y);
  status(moe_a2a_combine_send_compact(&s, expert_y.data_ptr(), ints(expert_meta), ints(expert_num_tokens),
                                      to_i32(std::min(rows_hint, capacity), "rows_hint"),
                                      to_i32(room, "compact_capacity_rows"), to_i32(capacity, "capacity_rows"),
                                      send_buf.data_ptr(), ints(send_meta), ints(send_counts),
                                      ints_or_null(send_back_plan), stream_of(stream)),
         "moe_a2a_combine_send_compact");
}
