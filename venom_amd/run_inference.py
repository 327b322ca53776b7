"""The reference's end-to-end sweep (end2end/run_inference.sh): BERT-large, GPT-2-large and the GPT-3-sized block,
each dense and with its linear layers in V:2:M for M in {8, 16, 32} and V in {64, 128}.  Prints the same CSV
(`algo,n,m,v,mean,median,std,len`; algo 0 = BERT, 1 = GPT-2, 2 = GPT-3 block) followed by one `#` summary line
per run.

    python -m venom_amd.run_inference [--repeats 10] [--models bert,gpt2,gpt3] [--fuse-ffn [--kernel-gelu]] [--merge-qkv] [--fuse-ln]"""
import argparse

from . import bert, gpt2, gpt3


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--repeats", type=int, default=10)
    ap.add_argument("--models", default="bert,gpt2,gpt3")
    ap.add_argument("--v", default="64,128")
    ap.add_argument("--m", default="8,16,32")
    ap.add_argument("--fuse-ffn", action="store_true", help="passed on to the three harnesses")
    ap.add_argument("--kernel-gelu", action="store_true", help="passed on to the three harnesses")
    ap.add_argument("--merge-qkv", action="store_true", help="passed on to the BERT harness (GPT-2's c_attn is one layer already)")
    ap.add_argument("--fuse-ln", action="store_true", help="passed on to the BERT harness (residual addition + LayerNorm as one kernel)")
    args = ap.parse_args(argv)
    extra = (["--fuse-ffn"] if args.fuse_ffn else []) + (["--kernel-gelu"] if args.kernel_gelu else [])
    print("algo,n,m,v,mean,median,std,len", flush=True)
    mains = {"bert": bert.main, "gpt2": gpt2.main, "gpt3": gpt3.main}
    for v in [int(x) for x in args.v.split(",")]:
        for name in args.models.split(","):
            for m in [int(x) for x in args.m.split(",")]:
                mains[name](["-m", str(m), "-n", "2", "-v", str(v), "--repeats", str(args.repeats)] + extra +
                            (["--merge-qkv"] if args.merge_qkv and name == "bert" else []) +
                            (["--fuse-ln"] if args.fuse_ln and name == "bert" else []))


if __name__ == "__main__":
    main()
