"""qil-amd (or python -m qil_amd) --model DIR --token-ids '[1, 2, 3]' --dtype bfloat16

Options and meanings follow the reference's command line (qil/__main__.py:8-21):
--model, --prompt | --token-ids, --device, --dtype, --max-new-tokens, --pages,
--page-size, --chunk-size, --output.  Its backend switches (--sdpa-backend,
--decode-attention) do not exist here.  Added: --token-budget, --max-active,
--temperature, --seed, --ignore-eos, and --random-config/--random-seed, which
write a random model folder into --model first.
"""
import argparse
import json
import sys
from pathlib import Path


def options():
    parser = argparse.ArgumentParser(prog='qil-amd', description=__doc__)
    parser.add_argument('--model', required=True, help='model folder (config.json + *.safetensors)')
    source = parser.add_mutually_exclusive_group(required=True)
    source.add_argument('--prompt', help='text; needs tokenizer.json in the model folder')
    source.add_argument('--token-ids', help='JSON list of token ids; no tokenizer needed')
    parser.add_argument('--device', default='cuda', choices=['cuda'])
    parser.add_argument('--dtype', default='float32', choices=['float32', 'bfloat16'])
    parser.add_argument('--max-new-tokens', default=64, type=int)
    parser.add_argument('--pages', default=256, type=int)
    parser.add_argument('--page-size', default=16, type=int)
    parser.add_argument('--chunk-size', default=64, type=int, help='prompt tokens per step and request')
    parser.add_argument('--token-budget', default=128, type=int, help='tokens per step over all requests')
    parser.add_argument('--max-active', default=4, type=int)
    parser.add_argument('--temperature', default=0.0, type=float, help='0 = greedy')
    parser.add_argument('--seed', default=0, type=int, help='seed of temperature sampling')
    parser.add_argument('--ignore-eos', action='store_true')
    parser.add_argument('--random-config', help='JSON file or string: write random weights for it into --model first')
    parser.add_argument('--random-seed', default=0, type=int)
    parser.add_argument('--output', type=Path)
    return parser


def prompt_tokens(args):
    """(token ids, decoder of token ids to text or None) from --token-ids or --prompt."""
    if args.token_ids is not None:
        return json.loads(args.token_ids), None
    from tokenizers import Tokenizer
    tokenizer = Tokenizer.from_file(str(Path(args.model) / 'tokenizer.json'))
    return (tokenizer.encode(args.prompt, add_special_tokens=False).ids,
            lambda ids: tokenizer.decode(ids, skip_special_tokens=True))


def main(argv=None):
    args = options().parse_args(argv)
    import torch
    from .engine import Engine
    from .weights import load_model, write_random_model
    if args.random_config:
        given = args.random_config
        source = given if given.lstrip().startswith('{') else Path(given).read_text()
        write_random_model(args.model, json.loads(source), args.random_seed)
    tokens, to_text = prompt_tokens(args)
    model = load_model(args.model, dtype=getattr(torch, args.dtype), device=args.device)
    engine = Engine(model, num_pages=args.pages, page_size=args.page_size, prefill_chunk=args.chunk_size,
                    token_budget=args.token_budget, max_active=args.max_active)
    try:
        report, = engine.generate([tokens], max_new_tokens=args.max_new_tokens, ignore_eos=args.ignore_eos,
                                  temperature=args.temperature, seed=args.seed)
    finally:
        engine.close()
    if to_text is not None:
        report['text'] = to_text(report['token_ids'])
    text = json.dumps(report, ensure_ascii=False, indent=2) + '\n'
    sys.stdout.write(text)
    if args.output is not None:
        args.output.parent.mkdir(parents=True, exist_ok=True)
        args.output.write_text(text)
    return 0


if __name__ == '__main__':
    sys.exit(main())
