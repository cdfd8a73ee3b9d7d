"""Greedy token IDs of a seeded random-init Whisper-base decoder loop: attention on the HIP kernels
must give the same IDs as attention on the CPU oracle.

The loop mirrors whisper_build_graph_decoder + whisper_decode_internal of the reference
(src/crispasr.cpp:3090-3300, 3412-3499): Q and K pre-scaled by hd^-0.25, new K/V rows copied
(F32 -> F16) into a [layer][ctx][n_state] cache, self-attention = FLASH_ATTN_EXT over strided
cache views with an F16 mask built from the cells (scale 1.0), cross-attention = FLASH_ATTN_EXT
over the encoder K/V zero-padded to a multiple of 256 rows with no mask (scale hd^-0.25).
Shape: the reference's test model header (models/for-tests-ggml-base.bin): 6 layers, 512 wide,
8 heads, vocab 51865, n_text_ctx 448, n_audio_ctx 1500.  Everything around attention (LN, matmul,
GELU) is the same torch code in both runs; only the attention backend differs.
"""
import numpy as np
import pytest
import torch

import crispasr_amd as ca
import oracle as ora

pytestmark = pytest.mark.gpu

N_LAYER, N_STATE, N_HEAD, N_VOCAB, N_TEXT_CTX, N_AUDIO_CTX = 6, 512, 8, 51865, 448, 1500
HD = N_STATE // N_HEAD
N_AUDIO_PAD = (N_AUDIO_CTX + 255) // 256 * 256          # GGML_PAD(n_audio_ctx, 256), src/crispasr.cpp:2733


def _randn(seed, *shape, std=1.0):
    return torch.from_numpy(ora.randn(seed, shape) * np.float32(std))


class Weights:
    def __init__(self, seed, dev):
        s = [seed * 1000]

        def nxt():
            s[0] += 1
            return s[0]

        lin = N_STATE ** -0.5
        self.te = _randn(nxt(), N_VOCAB, N_STATE, std=0.1).to(dev)
        self.pe = _randn(nxt(), N_TEXT_CTX, N_STATE, std=0.1).to(dev)
        self.layers = []
        for _ in range(N_LAYER):
            L = {}
            for name in ("q", "k", "v", "o", "cq", "co"):
                L[name + "_w"] = _randn(nxt(), N_STATE, N_STATE, std=1.5 * lin).to(dev)
                L[name + "_b"] = _randn(nxt(), N_STATE, std=0.1).to(dev)
            L["fc1_w"] = _randn(nxt(), 4 * N_STATE, N_STATE, std=lin).to(dev)
            L["fc1_b"] = _randn(nxt(), 4 * N_STATE, std=0.1).to(dev)
            L["fc2_w"] = _randn(nxt(), N_STATE, 4 * N_STATE, std=0.5 * lin).to(dev)
            L["fc2_b"] = _randn(nxt(), N_STATE, std=0.1).to(dev)
            for ln in ("ln0", "ln1", "ln2"):
                L[ln + "_w"] = (1.0 + _randn(nxt(), N_STATE, std=0.1)).to(dev)
                L[ln + "_b"] = _randn(nxt(), N_STATE, std=0.1).to(dev)
            # encoder memory of this layer, as whisper_encode leaves it in kv_cross: F16, K pre-scaled by
            # hd^-0.25 (src/crispasr.cpp:2940-2973), rows 1500..1535 zero
            kc = np.zeros((N_AUDIO_PAD, N_STATE), np.float32)
            vc = np.zeros((N_AUDIO_PAD, N_STATE), np.float32)
            kc[:N_AUDIO_CTX] = ora.randn(nxt(), (N_AUDIO_CTX, N_STATE)) * np.float32(HD ** -0.25)
            vc[:N_AUDIO_CTX] = ora.randn(nxt(), (N_AUDIO_CTX, N_STATE))
            L["kcross"] = ora.fp32_to_fp16(kc)
            L["vcross"] = ora.fp32_to_fp16(vc)
            self.layers.append(L)
        self.ln_w = (1.0 + _randn(nxt(), N_STATE, std=0.1)).to(dev)
        self.ln_b = _randn(nxt(), N_STATE, std=0.1).to(dev)


class GpuAttention:
    """K/V caches in device memory, attention through the C-ABI."""

    def __init__(self, w, n_ctx):
        self.n_ctx = n_ctx
        self.kv_k = ca.Tensor.empty(ca.F16, (N_STATE, n_ctx, N_LAYER))
        self.kv_v = ca.Tensor.empty(ca.F16, (N_STATE, n_ctx, N_LAYER))
        self.kv_k.buf.zero_()
        self.kv_v.buf.zero_()
        self.cross = [(ca.Tensor.from_host(L["kcross"], ca.F16, (HD, N_AUDIO_PAD, N_HEAD), (2, 2 * N_STATE, 2 * HD, 0)),
                       ca.Tensor.from_host(L["vcross"], ca.F16, (HD, N_AUDIO_PAD, N_HEAD), (2, 2 * N_STATE, 2 * HD, 0)))
                      for L in w.layers]
        self.kernels = set()

    @staticmethod
    def _wrap_q(x):          # [n_tok, n_state] f32 -> ne [hd, n_tok, n_head] view (ggml_permute of the reshape)
        n_tok = x.shape[0]
        return ca.Tensor(x.contiguous().view(torch.uint8).reshape(-1), ca.F32, (HD, n_tok, N_HEAD),
                         (4, 4 * N_STATE, 4 * HD, 4 * N_STATE * n_tok))

    def store_kv(self, il, kv_head, k, v):
        n_tok = k.shape[0]
        off = 2 * N_STATE * (il * self.n_ctx + kv_head)
        for cache, x in ((self.kv_k, k), (self.kv_v, v)):
            src = ca.Tensor(x.contiguous().view(torch.uint8).reshape(-1), ca.F32, (N_STATE, n_tok))
            ca.cpy(src, cache.view((n_tok * N_STATE,), (2, 0, 0, 0), off))      # ggml_view_1d + ggml_cpy

    def _fa(self, q, k, v, mask, scale):
        self.kernels.add(ca.ggml.flash_attn_plan(q, k, v, mask, scale)[0])
        out = ca.flash_attn_ext(q, k, v, mask, scale)
        n_tok = q.ne[1]
        return out.buf[: 4 * N_STATE * n_tok].view(torch.float32).reshape(n_tok, N_STATE)

    def self_attn(self, il, q, n_kv, mask_f16):
        nb = (2, 2 * N_STATE, 2 * HD, 0)
        off = 2 * N_STATE * self.n_ctx * il
        k = self.kv_k.view((HD, n_kv, N_HEAD), nb, off)
        v = self.kv_v.view((HD, n_kv, N_HEAD), nb, off)
        m = ca.Tensor.from_host(mask_f16, ca.F16, (n_kv, q.shape[0]))
        return self._fa(self._wrap_q(q), k, v, m, 1.0)

    def cross_attn(self, il, q):
        k, v = self.cross[il]
        return self._fa(self._wrap_q(q), k, v, None, HD ** -0.25)


class OracleAttention:
    """The same caches in host memory, attention on the CPU oracle."""

    def __init__(self, w, n_ctx, mode):
        self.n_ctx, self.mode = n_ctx, mode
        self.kv_k = np.zeros(N_LAYER * n_ctx * N_STATE * 2, np.uint8)
        self.kv_v = np.zeros(N_LAYER * n_ctx * N_STATE * 2, np.uint8)
        self.cross = [(ora.Tensor(L["kcross"].view(np.uint8).reshape(-1), ora.F16, (HD, N_AUDIO_PAD, N_HEAD), (2, 2 * N_STATE, 2 * HD, 0)),
                       ora.Tensor(L["vcross"].view(np.uint8).reshape(-1), ora.F16, (HD, N_AUDIO_PAD, N_HEAD), (2, 2 * N_STATE, 2 * HD, 0)))
                      for L in w.layers]

    @staticmethod
    def _wrap_q(x):
        n_tok = x.shape[0]
        raw = x.detach().cpu().contiguous().numpy().view(np.uint8).reshape(-1)
        return ora.Tensor(raw, ora.F32, (HD, n_tok, N_HEAD), (4, 4 * N_STATE, 4 * HD, 4 * N_STATE * n_tok))

    def store_kv(self, il, kv_head, k, v):
        n_tok = k.shape[0]
        off = 2 * N_STATE * (il * self.n_ctx + kv_head)
        for cache, x in ((self.kv_k, k), (self.kv_v, v)):
            src = ora.from_f32(x.detach().cpu().numpy().reshape(1, 1, n_tok, N_STATE))
            ora.cpy_f32(src, ora.Tensor(cache, ora.F16, (N_STATE, n_tok), None, off))

    def _fa(self, q, k, v, mask, scale, dev):
        out = ora.flash_attn_ext(q, k, v, mask, scale, mode=self.mode)       # [1, n_tok, H, hd]
        return torch.from_numpy(out.reshape(q.ne[1], N_STATE)).to(dev)

    def self_attn(self, il, q, n_kv, mask_f16):
        nb = (2, 2 * N_STATE, 2 * HD, 0)
        off = 2 * N_STATE * self.n_ctx * il
        k = ora.Tensor(self.kv_k, ora.F16, (HD, n_kv, N_HEAD), nb, off)
        v = ora.Tensor(self.kv_v, ora.F16, (HD, n_kv, N_HEAD), nb, off)
        m = ora.Tensor(mask_f16.view(np.uint8).reshape(-1).copy(), ora.F16, (n_kv, q.shape[0]))
        return self._fa(self._wrap_q(q), k, v, m, 1.0, q.device)

    def cross_attn(self, il, q):
        k, v = self.cross[il]
        return self._fa(self._wrap_q(q), k, v, None, HD ** -0.25, q.device)


def _ln(x, w, b):
    return torch.nn.functional.layer_norm(x, (N_STATE,), w, b, 1e-5)


def decode(w, attn, tokens, positions, cell_pos, cell_seq, seq_ids, kv_head):
    """One whisper_decode_internal call: tokens[i] at positions[i] for sequence seq_ids[i], written to
    cache cells kv_head.. ; returns logits [n_tok, n_vocab]."""
    n_tok = len(tokens)
    dev = w.te.device
    for i in range(n_tok):
        cell_pos[kv_head + i] = positions[i]
        cell_seq[kv_head + i] = seq_ids[i]
    n_kv = kv_head + n_tok
    # mask from the cells: -inf unless the cell belongs to the token's sequence and is not in its future
    mask = np.zeros((n_tok, n_kv), np.float32)
    for j in range(n_tok):
        for i in range(n_kv):
            if cell_seq[i] != seq_ids[j] or cell_pos[i] > positions[j]:
                mask[j, i] = -np.inf
    mask_f16 = ora.fp32_to_fp16(mask)
    x = w.te[torch.tensor(tokens, device=dev)] + w.pe[torch.tensor(positions, device=dev)]
    kq = HD ** -0.25
    for il, L in enumerate(w.layers):
        cur = _ln(x, L["ln0_w"], L["ln0_b"])
        q = (cur @ L["q_w"].T + L["q_b"]) * kq
        k = (cur @ L["k_w"].T) * kq
        v = cur @ L["v_w"].T + L["v_b"]
        attn.store_kv(il, kv_head, k, v)
        a = attn.self_attn(il, q, n_kv, mask_f16)
        x = x + a @ L["o_w"].T + L["o_b"]
        cur = _ln(x, L["ln1_w"], L["ln1_b"])
        q = cur @ L["cq_w"].T + L["cq_b"]
        a = attn.cross_attn(il, q)
        x = x + a @ L["co_w"].T + L["co_b"]
        cur = _ln(x, L["ln2_w"], L["ln2_b"])
        x = x + torch.nn.functional.gelu(cur @ L["fc1_w"].T + L["fc1_b"]) @ L["fc2_w"].T + L["fc2_b"]
    x = _ln(x, w.ln_w, w.ln_b)
    return x @ w.te.T


def greedy_loop(w, attn, prompt, n_steps, n_seq):
    """Prompt prefill for every sequence (one batch call, interleaved cells), then n_steps batched single-token
    steps, one token per sequence per step - the unified-cache layout of the reference's beam decoding."""
    n_ctx = attn.n_ctx
    cell_pos, cell_seq = [-1] * n_ctx, [-1] * n_ctx
    toks, pos, seq = [], [], []
    for p, t in enumerate(prompt):
        for s_ in range(n_seq):
            toks.append(t + s_)              # sequences differ from the first token on
            pos.append(p)
            seq.append(s_)
    logits = decode(w, attn, toks, pos, cell_pos, cell_seq, seq, 0)
    kv_head = len(toks)
    last = logits[-n_seq:]
    ids, margins = [], []
    for step in range(n_steps):
        top2 = torch.topk(last, 2, dim=-1)
        nxt = top2.indices[:, 0].tolist()
        margins.append(float((top2.values[:, 0] - top2.values[:, 1]).min()))
        ids.append(nxt)
        p = len(prompt) + step
        last = decode(w, attn, nxt, [p] * n_seq, cell_pos, cell_seq, list(range(n_seq)), kv_head)
        kv_head += n_seq
    return ids, margins


@pytest.mark.parametrize("n_seq", [1, 5])
def test_greedy_token_ids_match_the_cpu_run(n_seq):
    dev = torch.device("cuda")
    torch.backends.cuda.matmul.allow_tf32 = False
    w = Weights(7, dev)
    prompt, n_steps = [50258, 50259, 50359], 24
    n_ctx = 160
    print("whisper loop: n_seq", n_seq, flush=True)
    gpu = GpuAttention(w, n_ctx)
    ids_gpu, margins = greedy_loop(w, gpu, prompt, n_steps, n_seq)
    ids_cpu, _ = greedy_loop(w, OracleAttention(w, n_ctx, ora.MODE_EXACT), prompt, n_steps, n_seq)
    print("ids", ids_gpu[:6], "... min top-2 logit margin", min(margins), "kernels used", sorted(gpu.kernels), flush=True)
    assert ids_gpu == ids_cpu
    assert len({tuple(r) for r in ids_gpu}) > 1                       # the loop does move
    # the restatement of ggml-cpu's own arithmetic (f16 accumulator) lands on the same tokens
    ids_like, _ = greedy_loop(w, OracleAttention(w, n_ctx, ora.MODE_GGML_LIKE), prompt, n_steps, n_seq)
    assert ids_gpu == ids_like
    assert ca.ggml.KERNEL_DECODE_MMA in gpu.kernels
