#!/usr/bin/env python3
"""Interactive chat on the command line, in the manner of the reference's ``chat.py``.

Reference: chat.py — ``--model`` (required) and ``--system-prompt``; a session keeps the
history (system prompt first), turns it into tokens with the chat template
(``enable_thinking=True``), submits one request and prints the text of the new tokens after
every engine step; slash commands ``/help /clear /exit /history /settings /maxtokens N
/top-k N /top-p F /temperature F /system TEXT``. ``/reset`` is listed in the reference's help
but not implemented there; here it clears the history and restores the system prompt.
"""
import argparse
import os
import sys
from typing import Generator, List

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HELP = """
Commands:
/help     - Show this help message
/clear    - Clear conversation history
/exit     - Exit the chat
/reset    - Reset and clear history
/history  - Show conversation history

Settings:
/settings             - Show current settings
/maxtokens <num>      - Set max tokens for response
/top-k <num>          - Set top-k sampling value
/top-p <float>        - Set top-p sampling value
/temperature <float>  - Set temperature for sampling
/system <text>        - Set system prompt
"""


class ChatSession:
    def __init__(self, llm, system_prompt: str = None, sampling_params=None):
        from minivllm_amd import SamplingParams
        self.llm = llm
        self.system_prompt = system_prompt or "You are a helpful assistant."
        self.sampling_params = sampling_params or SamplingParams()
        self.history: List[dict] = [{"role": "system", "content": self.system_prompt}]

    def build_model_input_tokens(self, user_message: str) -> List[int]:
        messages = self.history + [{"role": "user", "content": user_message}]
        return self.llm.tokenizer.apply_chat_template(messages, tokenize=True, add_generation_prompt=True,
                                                      enable_thinking=True)

    def run_command(self, command: str, args: List[str]) -> None:
        sp = self.sampling_params
        if command == "/help":
            print(HELP)
        elif command == "/clear":
            self.history = []
            print("\n[Conversation history cleared]\n")
        elif command == "/reset":
            self.history = [{"role": "system", "content": self.system_prompt}]
            print("\n[Conversation reset]\n")
        elif command == "/history":
            self.print_history()
        elif command == "/system":
            if not args:
                print("\n[Usage: /system <system prompt text>]\n")
                return
            self.system_prompt = " ".join(args)
            self.history = [{"role": "system", "content": self.system_prompt}]
            print(f"\n[System prompt set to: {self.system_prompt}]\n")
        elif command == "/maxtokens":
            if len(args) != 1 or not args[0].isdigit() or int(args[0]) < 1:
                print("\n[Usage: /maxtokens <num>]\n")
                return
            sp.max_tokens = int(args[0])
            print(f"\n[Max tokens set to {sp.max_tokens}]\n")
        elif command == "/top-k":
            if len(args) != 1 or not args[0].isdigit():
                print("\n[Usage: /top-k <num>]\n")
                return
            sp.top_k = int(args[0])
            print(f"\n[Top-k set to {sp.top_k}]\n")
        elif command == "/top-p":
            try:
                value = float(args[0])
                if not (0.0 < value <= 1.0):
                    raise ValueError
                sp.top_p = value
                print(f"\n[Top-p set to {sp.top_p}]\n")
            except (ValueError, IndexError):
                print("\n[Usage: /top-p <float in (0, 1]>]\n")
        elif command == "/temperature":
            try:
                value = float(args[0])
                if value < 0:
                    raise ValueError
                sp.temperature = value
                print(f"\n[Temperature set to {sp.temperature}]\n")
            except (ValueError, IndexError):
                print("\n[Usage: /temperature <float >= 0>]\n")
        elif command == "/settings":
            self.print_settings()
        else:
            print(f"\n[Unknown command: {command}. Type /help for available commands]\n")

    def print_history(self) -> None:
        if not self.history:
            print("\n[No conversation history]\n")
            return
        print("\n" + "=" * 60 + "\nConversation History:\n" + "=" * 60)
        for msg in self.history:
            print(f"\n{msg['role'].capitalize()}: {msg['content']}")
        print("=" * 60 + "\n")

    def print_settings(self) -> None:
        sp = self.sampling_params
        print("\nCurrent Settings:")
        print(f"Max Tokens: {sp.max_tokens}\nTop-k: {sp.top_k}\nTop-p: {sp.top_p}\nTemperature: {sp.temperature}\n")
        print(f"System Prompt: {self.system_prompt}\n")

    def generate(self, prompt: List[int]) -> Generator[str, None, None]:
        """Submits the prompt and yields the text of the tokens each engine step adds."""
        req = self.llm.submit(prompt, self.sampling_params)
        seen = req.prompt_token_count
        while not req.finished:
            self.llm.step()
            new = req.tokens[seen:]
            seen = len(req.tokens)
            if new:
                yield self.llm.tokenizer.decode(new, skip_special_tokens=True)

    def start(self) -> None:
        print("\n=== mini-vllm_amd interactive chat ===\n\nType your message and press Enter to chat.\n"
              "Type /help for available commands.\nType /exit to exit.\n")
        self.print_settings()
        while True:
            try:
                user_input = input("You: ").strip()
            except (KeyboardInterrupt, EOFError):
                print("\n\nGoodbye!\n")
                break
            if not user_input:
                continue
            if user_input.startswith("/"):
                items = user_input.split()
                if items[0].lower() == "/exit":
                    print("\nGoodbye!\n")
                    break
                self.run_command(items[0].lower(), items[1:])
                continue
            try:
                tokens = self.build_model_input_tokens(user_input)
                print("Assistant: ", end="", flush=True)
                response = ""
                for text in self.generate(tokens):
                    print(text, end="", flush=True)
                    response += text
                print("\n\n" + "=" * 80 + "\n")
                self.history.append({"role": "user", "content": user_input})
                self.history.append({"role": "assistant", "content": response.strip()})
            except KeyboardInterrupt:
                print("\n\nGoodbye!\n")
                break
            except ValueError as e:          # e.g. the conversation outgrew max_model_len
                print(f"\n[{e}]\n")


def main() -> int:
    from run import add_engine_options, engine_config_from
    ap = argparse.ArgumentParser(description="mini-vllm_amd interactive chat")
    add_engine_options(ap)
    for action in ap._actions:               # the reference requires --model (chat.py:236)
        if action.dest == "model":
            action.required, action.default = True, None
    ap.add_argument("--system-prompt", type=str, default="You are a helpful assistant.",
                    help="System prompt for the chat session")
    args = ap.parse_args()
    if not os.path.isdir(args.model):
        ap.error(f"--model {args.model!r} is not a directory")
    print(f"Loading model: {args.model}...")
    from minivllm_amd import LLM
    llm = LLM(config=engine_config_from(args))
    if llm.tokenizer is None:
        print("this model folder has no tokenizer; chat needs one", file=sys.stderr)
        return 2
    print("Model loaded successfully!\n")
    ChatSession(llm, system_prompt=args.system_prompt).start()
    return 0


if __name__ == "__main__":
    sys.exit(main())
