"""CPU checkers for the signature path.  Test infrastructure only: the shipped package never imports this."""
