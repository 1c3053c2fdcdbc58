"""python -m spy_amd.cli MODEL.gguf -p "prompt" -n 32

The token loop of Spy's command line (app/cli/include/cli.h:60-129 in the Spy tree) on the HIP backend: the
prompt is tokenized with the file's SentencePiece vocabulary (BOS added), passed through the model, and
n tokens are sampled greedily on the device and printed as text with the timings the reference prints
(prompt tokens per second, generated tokens per second)."""
import argparse
import sys
import time


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[1])
    ap.add_argument("model", help="GGUF file (LLaMA architecture, Q4_0 / Q8_0 / Q4_K / Q6_K matrices)")
    ap.add_argument("-p", "--prompt", default="Once upon a time")
    ap.add_argument("-n", "--n-predict", type=int, default=32)
    ap.add_argument("-c", "--ctx", type=int, default=0, help="context to allocate (0: the file's context_length)")
    ap.add_argument("--exact", action="store_true",
                    help="exact-order mode: every float sum in the order of Spy's host backend, so that logits and tokens are the CPU backend's bit for bit (slow)")
    args = ap.parse_args(argv)
    from . import gguf as G
    import numpy as np
    if args.exact:
        from . import _lib
        _lib.load().spy_hip_set_exact_order(1)
    m = G.GGUFModel(args.model, n_ctx=args.ctx)
    print("loaded %.2f GB: parse %.1f ms, upload %.0f ms, set-up %.0f ms" % (m.weight_bytes / 1e9, m.parse_ms, m.upload_ms, m.create_ms), file=sys.stderr)
    ids = m.vocab.tokenize(args.prompt, add_bos=True, special=False)
    if len(ids) + args.n_predict > m.desc.n_ctx:
        sys.exit("prompt (%d tokens) + %d new tokens do not fit the context of %d" % (len(ids), args.n_predict, m.desc.n_ctx))
    t0 = time.perf_counter()
    logits = m.engine.forward(np.asarray(ids, dtype=np.int32), 0)
    t1 = time.perf_counter()
    first = int(np.argmax(logits[-1]))
    new = [first] + ([int(t) for t in m.engine.decode_greedy(first, len(ids), args.n_predict - 1)] if args.n_predict > 1 else [])
    t2 = time.perf_counter()
    sys.stdout.write(args.prompt + m.vocab.detokenize(new).decode("utf-8", "replace") + "\n")
    print("prompt: %d tokens, %.1f tok/s; generation: %d tokens, %.1f tok/s" %
          (len(ids), len(ids) / (t1 - t0), len(new), len(new) / max(t2 - t1, 1e-9)), file=sys.stderr)
    m.close()


if __name__ == "__main__":
    main()
