
<bos><eos><end_of_turn>